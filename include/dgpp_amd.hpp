// C++ face of the C ABI (dgpp_amd.h): the reference's `dgpp::launch_*` free functions with their
// own names, argument order, default arguments and error behaviour (std::invalid_argument for a
// refused call, std::runtime_error for a failed runtime call), so host code written against
// src/kernels/glm_moe_launch.hpp, fp4_gemv.hpp, scale_gemm.hpp, fp8_dequant.hpp and minimax.hpp
// compiles against this header with `cudaStream_t` replaced by `hipStream_t`. Header-only.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "dgpp_amd.h"

namespace dgpp {

using MoeExpertView = DgppMoeExpertView;   // src/models/glm/moe.hpp:232
using MoeSegment = DgppMoeSegment;         // src/kernels/glm_moe_launch.hpp:67
using MoeTile = DgppMoeTile;               // src/kernels/glm_moe_launch.hpp:151
using GlmFp4Matrix = DgppFp4Matrix;        // src/models/quant_matrix.hpp:117
using Fp8GemvProblem = DgppFp8GemvProblem; // src/kernels/scale_gemm.hpp:85

// The device code reads these by offset: the sizes are part of the ABI.
static_assert(sizeof(MoeExpertView) == 96 && sizeof(MoeSegment) == 12 && sizeof(MoeTile) == 8 &&
                  sizeof(GlmFp4Matrix) == 56,
              "POD layouts shared with the kernels");

constexpr int kFp4Group = 16;
constexpr int kMxfp4Group = 32;

// src/models/quant_matrix.hpp:16-47 (the fields the path reads).
struct GlmQuantMatrix {
  const uint8_t* payload = nullptr;
  const float* scales = nullptr;
  const uint8_t* scales_e8m0 = nullptr;
  int64_t rows = 0;
  int64_t cols = 0;
  int scale_block_rows = 128;
  int scale_block_cols = 128;
};

enum class MoeRouterMode { SigmoidBias = 0, SoftmaxTopk = 1, SqrtSoftplusBias = 2 };

// src/models/glm/moe.hpp:51-134 (the fields the path reads).
struct GlmMoeConfig {
  int hidden = 4096;
  int inter = 2048;
  int n_experts = 288;
  int top_k = 8;
  int n_shared_experts = 1;
  float routed_scaling_factor = 2.5f;
  bool norm_topk_prob = true;
  float swiglu_limit = 10.0f;
  bool shared_slots_early = false;
  MoeRouterMode router_mode = MoeRouterMode::SigmoidBias;

  DgppMoeConfig c_config() const {
    return DgppMoeConfig{hidden, inter, n_experts, top_k, n_shared_experts, routed_scaling_factor,
                         norm_topk_prob ? 1 : 0, swiglu_limit, static_cast<int32_t>(router_mode)};
  }
  static void validate_config(const GlmMoeConfig& c);
};

namespace detail {
inline void check(int rc) {
  if (rc == DGPP_OK) return;
  const std::string msg = dgpp_last_error();
  if (rc == DGPP_INVALID_ARGUMENT) throw std::invalid_argument(msg);
  throw std::runtime_error(msg);
}
inline int shift_of(int block) {
  int s = 0;
  while ((1 << s) < block) ++s;
  return s;
}
}  // namespace detail

inline void GlmMoeConfig::validate_config(const GlmMoeConfig& c) {
  const DgppMoeConfig cc = c.c_config();
  detail::check(dgpp_moe_config_validate(&cc));
}

// MoeExpertView::of (src/models/glm/moe.hpp:248-256)
inline MoeExpertView expert_view_of(const GlmQuantMatrix& m) {
  MoeExpertView v{};
  v.payload = m.payload;
  v.scales = m.scales;
  v.scale_shift_rows = detail::shift_of(m.scale_block_rows);
  v.scale_shift_cols = detail::shift_of(m.scale_block_cols);
  v.fp4_group = kFp4Group;
  return v;
}
inline MoeExpertView expert_view_of(const GlmFp4Matrix& m) {
  MoeExpertView v{};
  v.payload = m.payload;
  v.fp4_scales = m.scales;
  v.fp4_global = m.global_scale;
  v.scale_shift_rows = 7;
  v.scale_shift_cols = 7;
  v.fp4_group = m.scale_group;
  return v;
}

// ---- src/kernels/glm_moe_launch.hpp ---------------------------------------------------------------
inline void launch_moe_router(const uint16_t* hidden, const uint16_t* gate, const float* bias, int32_t* ids,
                              float* weights, float* scores, float* biased, const GlmMoeConfig& cfg, int tokens,
                              hipStream_t stream, int* counters = nullptr, bool allow_tiled = true) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_router(hidden, gate, bias, ids, weights, scores, biased, &c, tokens, stream, counters,
                                       allow_tiled ? 1 : 0));
}
inline void launch_moe_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int32_t* ids,
                                   float* weights, const GlmMoeConfig& cfg, int vocab, int n_tokens, hipStream_t stream) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_hash_routes(tokens, tid2eid, scores, ids, weights, &c, vocab, n_tokens, stream));
}
// The selection half alone (src/kernels/glm_moe.cu:314-329).
inline void launch_moe_router_select(const float* scores, const float* biased, int32_t* ids, float* weights,
                                     const GlmMoeConfig& cfg, int tokens, hipStream_t stream) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_router_select(scores, biased, ids, weights, &c, tokens, stream));
}
// Extension: selection + slot order in one launch (see dgpp_amd.h).
inline void launch_moe_router_select_order(const float* scores, const float* biased, int32_t* ids, float* weights,
                                           int32_t* order, const GlmMoeConfig& cfg, int tokens, hipStream_t stream,
                                           bool shared_early = false) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_router_select_order(scores, biased, ids, weights, order, &c, tokens,
                                                    shared_early ? 1 : 0, stream));
}
// Extension: the router's score rows without the selection (see dgpp_amd.h).
inline void launch_moe_router_dots(const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                                   float* biased, const GlmMoeConfig& cfg, int tokens, hipStream_t stream) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_router_dots(hidden, gate, bias, scores, biased, &c, tokens, stream));
}
// Extension: selection + routed gate/up in one launch (see dgpp_amd.h).
inline void launch_moe_select_gate_up_swiglu(const float* scores, const float* biased, int32_t* ids, float* weights,
                                             const GlmMoeConfig& cfg, int tokens, const uint16_t* x, size_t x_stride,
                                             const MoeExpertView* views, int n_routed, int k_routed, uint16_t* act,
                                             int act_stride, float limit, hipStream_t stream) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_select_gate_up_swiglu(scores, biased, ids, weights, &c, tokens, x, x_stride, views, n_routed,
                                                      k_routed, act, act_stride, limit, stream));
}
inline void launch_moe_select_gate_up_swiglu_fp4(const float* scores, const float* biased, int32_t* ids, float* weights,
                                                 const GlmMoeConfig& cfg, int tokens, const uint16_t* x, size_t x_stride,
                                                 const MoeExpertView* views, int n_routed, int k_routed, uint16_t* act,
                                                 int act_stride, float limit, hipStream_t stream, int fp4_group = 16) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_select_gate_up_swiglu_fp4(scores, biased, ids, weights, &c, tokens, x, x_stride, views,
                                                          n_routed, k_routed, act, act_stride, limit, stream, fp4_group));
}
inline void launch_moe_swiglu_clamp(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, float limit,
                                    hipStream_t stream) {
  detail::check(dgpp_launch_moe_swiglu_clamp(gate, up, out, n, limit, stream));
}
inline void launch_moe_gather_rows(const uint16_t* src, const int32_t* rows, uint16_t* dst, int n_rows, int hidden,
                                   hipStream_t stream) {
  detail::check(dgpp_launch_moe_gather_rows(src, rows, dst, n_rows, hidden, stream));
}
inline void launch_moe_accum(float* acc, const float* y, const int32_t* rows, const float* row_weights, int n_rows,
                             int hidden, hipStream_t stream) {
  detail::check(dgpp_launch_moe_accum(acc, y, rows, row_weights, n_rows, hidden, stream));
}
inline void launch_moe_round_bf16(uint16_t* out, const float* acc, int64_t n, hipStream_t stream) {
  detail::check(dgpp_launch_moe_round_bf16(out, acc, n, stream));
}
inline void launch_moe_segment(const int32_t* ids, int tokens, int top_k, int n_experts, int32_t* rows,
                               int32_t* slot_row, MoeSegment* segs, hipStream_t stream) {
  detail::check(dgpp_launch_moe_segment(ids, tokens, top_k, n_experts, rows, slot_row, segs, stream));
}
inline int moe_tile_list_capacity(int n_segs, int total_rows, int tile_rows) {
  return dgpp_moe_tile_list_capacity(n_segs, total_rows, tile_rows);
}
inline void launch_moe_tile_list(const MoeSegment* segs, int n_segs, int tile_rows, MoeTile* tiles, int32_t* count,
                                 hipStream_t stream) {
  detail::check(dgpp_launch_moe_tile_list(segs, n_segs, tile_rows, tiles, count, stream));
}
inline int moe_run_groups_max(int slots) { return dgpp_moe_run_groups_max(slots); }
inline void launch_moe_slot_order(const int32_t* ids, int32_t* order, int slots, int top_k, int n_experts,
                                  hipStream_t stream, bool shared_early = false, int32_t* runs = nullptr) {
  detail::check(dgpp_launch_moe_slot_order(ids, order, slots, top_k, n_experts, stream, shared_early ? 1 : 0, runs));
}
inline void launch_moe_accum_ordered(uint16_t* out, const float* down, size_t down_stride, const int32_t* slot_row,
                                     const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                                     int top_k, int hidden, hipStream_t stream) {
  detail::check(dgpp_launch_moe_accum_ordered(out, down, down_stride, slot_row, slot_ids, slot_w, shared_row0, tokens,
                                              top_k, hidden, stream));
}
inline void launch_moe_accum_ordered_f32(float* out, const float* down, size_t down_stride, const int32_t* slot_row,
                                         const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                                         int top_k, int hidden, hipStream_t stream) {
  detail::check(dgpp_launch_moe_accum_ordered_f32(out, down, down_stride, slot_row, slot_ids, slot_w, shared_row0,
                                                  tokens, top_k, hidden, stream));
}
inline void launch_moe_accum_ordered_bf16down(uint16_t* out, const uint16_t* down, size_t down_stride, const int32_t* slot_row,
                                              const int32_t* slot_ids, const float* slot_w, int tokens, int top_k, int hidden,
                                              hipStream_t stream) {
  detail::check(dgpp_launch_moe_accum_ordered_bf16down(out, down, down_stride, slot_row, slot_ids, slot_w, tokens, top_k, hidden,
                                                       stream));
}
inline void launch_moe_accum_ordered_f32_bf16down(float* out, const uint16_t* down, size_t down_stride, const int32_t* slot_row,
                                                  const int32_t* slot_ids, const float* slot_w, int tokens, int top_k,
                                                  int hidden, hipStream_t stream) {
  detail::check(dgpp_launch_moe_accum_ordered_f32_bf16down(out, down, down_stride, slot_row, slot_ids, slot_w, tokens, top_k,
                                                           hidden, stream));
}
inline void launch_moe_slot_accum(uint16_t* out, const float* contrib, const float* weights, int tokens, int hidden,
                                  int top_k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_slot_accum(out, contrib, weights, tokens, hidden, top_k, stream));
}
inline void launch_moe_slot_accum_routed_f32(float* out, const float* contrib, const float* weights, int tokens,
                                             int hidden, int top_k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_slot_accum_routed_f32(out, contrib, weights, tokens, hidden, top_k, stream));
}
// launch_moe_slot_accum_routed_f32 + launch_moe_round_bf16 in one launch (no reference counterpart).
inline void launch_moe_slot_accum_routed_bf16(uint16_t* out, const float* contrib, const float* weights, int tokens,
                                              int hidden, int top_k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_slot_accum_routed_bf16(out, contrib, weights, tokens, hidden, top_k, stream));
}
inline void launch_moe_slot_gate_up_swiglu(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                           const MoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                           int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                           const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                           int act_stride, int slots, int top_k, float limit, hipStream_t stream,
                                           int sh_rs = 7, int sh_cs = 7) {
  detail::check(dgpp_launch_moe_slot_gate_up_swiglu(x, x_stride, ids, order, views, n_routed, k_routed, n_shared,
                                                    k_shared, sh_gate_payload, sh_gate_scales, sh_up_payload,
                                                    sh_up_scales, act, act_stride, slots, top_k, limit, stream, sh_rs,
                                                    sh_cs));
}
inline void launch_moe_slot_down(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                 const MoeExpertView* views, int n_routed, int k_routed, int n_shared, int k_shared,
                                 const uint8_t* sh_payload, const float* sh_scales, float* out, int out_stride,
                                 int slots, int top_k, hipStream_t stream, int sh_rs = 7, int sh_cs = 7) {
  detail::check(dgpp_launch_moe_slot_down(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                          sh_payload, sh_scales, out, out_stride, slots, top_k, stream, sh_rs, sh_cs));
}
inline void launch_moe_slot_gate_up_swiglu_fp4(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                               const int32_t* order, const MoeExpertView* views, int n_routed,
                                               int k_routed, int n_shared, int k_shared,
                                               const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                               const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                               int act_stride, int slots, int top_k, float limit, hipStream_t stream,
                                               int shared_view_base = -1, int fp4_group = 16, int sh_rs = 7,
                                               int sh_cs = 7) {
  detail::check(dgpp_launch_moe_slot_gate_up_swiglu_fp4(x, x_stride, ids, order, views, n_routed, k_routed, n_shared,
                                                        k_shared, sh_gate_payload, sh_gate_scales, sh_up_payload,
                                                        sh_up_scales, act, act_stride, slots, top_k, limit, stream,
                                                        shared_view_base, fp4_group, sh_rs, sh_cs));
}
inline void launch_moe_slot_gate_up_swiglu_mixed(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                                 const MoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                                 int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                                 const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                                 int act_stride, int slots, int top_k, float limit, bool gate_fp4,
                                                 int fp4_group, hipStream_t stream, int sh_rs = 7, int sh_cs = 7) {
  detail::check(dgpp_launch_moe_slot_gate_up_swiglu_mixed(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                                          sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act,
                                                          act_stride, slots, top_k, limit, gate_fp4 ? 1 : 0, fp4_group, stream,
                                                          sh_rs, sh_cs));
}
inline void launch_moe_slot_down_fp4(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                     const MoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                     int k_shared, const uint8_t* sh_payload, const float* sh_scales, float* out,
                                     int out_stride, int slots, int top_k, hipStream_t stream,
                                     int shared_view_base = -1, int fp4_group = 16, int sh_rs = 7, int sh_cs = 7,
                                     int* tile_counter = nullptr) {
  detail::check(dgpp_launch_moe_slot_down_fp4(act, act_stride, ids, order, views, n_routed, k_routed, n_shared,
                                              k_shared, sh_payload, sh_scales, out, out_stride, slots, top_k, stream,
                                              shared_view_base, fp4_group, sh_rs, sh_cs, tile_counter));
}
// Extensions: the four decode-slot launchers with the pass selector (1 routed, 2 shared, 3 both) and, for the down
// launchers, the accumulation the shared pass ends with, as trailing arguments (see dgpp_amd.h).
inline void launch_moe_slot_gate_up_swiglu_ex(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                              const MoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                              int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                              const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                              int act_stride, int slots, int top_k, float limit, hipStream_t stream,
                                              int sh_rs, int sh_cs, int passes) {
  detail::check(dgpp_launch_moe_slot_gate_up_swiglu_ex(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                                       sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act,
                                                       act_stride, slots, top_k, limit, stream, sh_rs, sh_cs, passes));
}
inline void launch_moe_slot_down_ex(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                    const MoeExpertView* views, int n_routed, int k_routed, int n_shared, int k_shared,
                                    const uint8_t* sh_payload, const float* sh_scales, float* out, int out_stride,
                                    int slots, int top_k, hipStream_t stream, int sh_rs, int sh_cs, int passes,
                                    const float* acc_weights, uint16_t* acc_out) {
  detail::check(dgpp_launch_moe_slot_down_ex(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                             sh_payload, sh_scales, out, out_stride, slots, top_k, stream, sh_rs, sh_cs,
                                             passes, acc_weights, acc_out));
}
inline void launch_moe_slot_gate_up_swiglu_fp4_ex(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                                  const int32_t* order, const MoeExpertView* views, int n_routed,
                                                  int k_routed, int n_shared, int k_shared,
                                                  const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                                  const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                                  int act_stride, int slots, int top_k, float limit, hipStream_t stream,
                                                  int shared_view_base, int fp4_group, int sh_rs, int sh_cs, int passes) {
  detail::check(dgpp_launch_moe_slot_gate_up_swiglu_fp4_ex(x, x_stride, ids, order, views, n_routed, k_routed, n_shared,
                                                           k_shared, sh_gate_payload, sh_gate_scales, sh_up_payload,
                                                           sh_up_scales, act, act_stride, slots, top_k, limit, stream,
                                                           shared_view_base, fp4_group, sh_rs, sh_cs, passes));
}
inline void launch_moe_slot_down_fp4_ex(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                        const MoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                        int k_shared, const uint8_t* sh_payload, const float* sh_scales, float* out,
                                        int out_stride, int slots, int top_k, hipStream_t stream, int shared_view_base,
                                        int fp4_group, int sh_rs, int sh_cs, int* tile_counter, int passes,
                                        const float* acc_weights, uint16_t* acc_out) {
  detail::check(dgpp_launch_moe_slot_down_fp4_ex(act, act_stride, ids, order, views, n_routed, k_routed, n_shared,
                                                 k_shared, sh_payload, sh_scales, out, out_stride, slots, top_k, stream,
                                                 shared_view_base, fp4_group, sh_rs, sh_cs, tile_counter, passes,
                                                 acc_weights, acc_out));
}
// Extensions: routed down rows + ordered accumulation in one token-major launch (see dgpp_amd.h).
inline void launch_moe_slot_down_accum(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                       const MoeExpertView* views, int n, int k, int tokens, int top_k,
                                       const float* weights, uint16_t* out_bf16, float* out_f32, hipStream_t stream) {
  detail::check(dgpp_launch_moe_slot_down_accum(act, act_stride, ids, views, n, k, tokens, top_k, weights, out_bf16,
                                                out_f32, stream));
}
inline void launch_moe_slot_down_accum_fp4(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                           const MoeExpertView* views, int n, int k, int tokens, int top_k,
                                           const float* weights, uint16_t* out_bf16, float* out_f32, hipStream_t stream,
                                           int fp4_group = kFp4Group) {
  detail::check(dgpp_launch_moe_slot_down_accum_fp4(act, act_stride, ids, views, n, k, tokens, top_k, weights, out_bf16,
                                                    out_f32, stream, fp4_group));
}
inline size_t moe_slot_chain_ready_bytes(int tokens, int top_k) { return dgpp_moe_slot_chain_ready_bytes(tokens, top_k); }
inline void launch_moe_slot_chain(const uint16_t* x, size_t x_stride, const int32_t* ids, const MoeExpertView* views, int inter,
                                  int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                                  const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                  hipStream_t stream, unsigned spins = 0) {
  detail::check(dgpp_launch_moe_slot_chain(x, x_stride, ids, views, inter, hidden, act, act_stride, tokens, top_k, limit,
                                           weights, out_bf16, out_f32, ready, status, spins, stream));
}
inline void launch_moe_slot_chain_fp4(const uint16_t* x, size_t x_stride, const int32_t* ids, const MoeExpertView* views,
                                      int inter, int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                                      const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                      hipStream_t stream, int fp4_group = kFp4Group, unsigned spins = 0) {
  detail::check(dgpp_launch_moe_slot_chain_fp4(x, x_stride, ids, views, inter, hidden, act, act_stride, tokens, top_k, limit,
                                               weights, out_bf16, out_f32, ready, status, spins, stream, fp4_group));
}
inline void launch_moe_select_slot_chain(const float* scores, const float* biased, int32_t* ids, float* weights,
                                         const GlmMoeConfig& cfg, int tokens, const uint16_t* x, size_t x_stride,
                                         const MoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride,
                                         float limit, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                         hipStream_t stream, unsigned spins = 0) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_select_slot_chain(scores, biased, ids, weights, &c, tokens, x, x_stride, views, inter, hidden, act,
                                                  act_stride, limit, out_bf16, out_f32, ready, status, spins, stream));
}
inline void launch_moe_select_slot_chain_fp4(const float* scores, const float* biased, int32_t* ids, float* weights,
                                             const GlmMoeConfig& cfg, int tokens, const uint16_t* x, size_t x_stride,
                                             const MoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride,
                                             float limit, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                             hipStream_t stream, int fp4_group = kFp4Group, unsigned spins = 0) {
  const DgppMoeConfig c = cfg.c_config();
  detail::check(dgpp_launch_moe_select_slot_chain_fp4(scores, biased, ids, weights, &c, tokens, x, x_stride, views, inter, hidden,
                                                      act, act_stride, limit, out_bf16, out_f32, ready, status, spins, stream,
                                                      fp4_group));
}
inline void launch_moe_grouped_gemv_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                         int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                         uint16_t* out, size_t out_stride, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_grouped_gemv_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which,
                                                  out, out_stride, n, k, stream));
}
inline void launch_moe_grouped_gemv_f32(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                        int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                        float* out, size_t out_stride, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_grouped_gemv_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which,
                                                 out, out_stride, n, k, stream));
}
inline void launch_moe_grouped_gemv_fp4_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                             int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                             uint16_t* out, size_t out_stride, int n, int k, hipStream_t stream,
                                             int fp4_group = 16) {
  detail::check(dgpp_launch_moe_grouped_gemv_fp4_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views,
                                                      which, out, out_stride, n, k, stream, fp4_group));
}
inline void launch_moe_grouped_gemv_fp4_f32(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                            int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                            float* out, size_t out_stride, int n, int k, hipStream_t stream,
                                            int fp4_group = 16) {
  detail::check(dgpp_launch_moe_grouped_gemv_fp4_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views,
                                                     which, out, out_stride, n, k, stream, fp4_group));
}

// ---- src/kernels/minimax.hpp:11 -----------------------------------------------------------------------
inline void minimax_router(const uint16_t* x, const float* gate, const float* bias, int rows, int hidden, int experts, int topk,
                           float factor, float* scores, int32_t* ids, float* weights, hipStream_t stream) {
  detail::check(dgpp_minimax_router(x, gate, bias, rows, hidden, experts, topk, factor, scores, ids, weights, stream));
}
inline void minimax_compact_segments(const MoeSegment* input, MoeSegment* output, int experts, int capacity,
                                     hipStream_t stream) {
  detail::check(dgpp_minimax_compact_segments(input, output, experts, capacity, stream));
}

// ---- src/kernels/fp4_gemv.hpp ---------------------------------------------------------------------------
inline void launch_fp4_gemv_bf16(const uint16_t* act, size_t act_row_stride_elems, const GlmFp4Matrix& w,
                                 uint16_t* out, int m, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_fp4_gemv_bf16(act, act_row_stride_elems, &w, out, m, n, k, stream));
}
inline void launch_fp4_gemv_f32(const uint16_t* act, size_t act_row_stride_elems, const GlmFp4Matrix& w, float* out,
                                int m, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_fp4_gemv_f32(act, act_row_stride_elems, &w, out, m, n, k, stream));
}
inline bool fp4_gemv_accepts(const GlmFp4Matrix& w) { return dgpp_fp4_gemv_accepts(&w) != 0; }

// ---- matrix-core launchers: src/kernels/glm_moe_launch.hpp:103-125, :311-345; src/kernels/mma_gemv.hpp:65-85 ----
inline void launch_dense_mma_bf16(const uint16_t* act, size_t act_stride, const uint8_t* payload, const float* scales,
                                  uint16_t* out, int m, int n, int k, hipStream_t stream, size_t out_stride = 0) {
  detail::check(dgpp_launch_dense_mma_bf16(act, act_stride, payload, scales, out, m, n, k, stream, out_stride));
}
inline void launch_dense_mma_f32(const uint16_t* act, size_t act_stride, const uint8_t* payload, const float* scales,
                                 float* out, int m, int n, int k, hipStream_t stream, size_t out_stride = 0) {
  detail::check(dgpp_launch_dense_mma_f32(act, act_stride, payload, scales, out, m, n, k, stream, out_stride));
}
inline void launch_dense_mma_fp4_bf16(const uint16_t* act, size_t act_stride, const GlmFp4Matrix& w, uint16_t* out, int m,
                                      int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_dense_mma_fp4_bf16(act, act_stride, &w, out, m, n, k, stream));
}
inline void launch_dense_mma_fp4_f32(const uint16_t* act, size_t act_stride, const GlmFp4Matrix& w, float* out, int m, int n,
                                     int k, hipStream_t stream) {
  detail::check(dgpp_launch_dense_mma_fp4_f32(act, act_stride, &w, out, m, n, k, stream));
}
inline void launch_mma_gemv_fp4_bf16(const uint16_t* act, size_t act_stride, const GlmFp4Matrix& w, uint16_t* out, int m,
                                     int n, int k, size_t out_stride, hipStream_t stream, void* ws = nullptr,
                                     size_t ws_bytes = 0) {
  detail::check(dgpp_launch_mma_gemv_fp4_bf16(act, act_stride, &w, out, m, n, k, out_stride, stream, ws, ws_bytes));
}
// The same on the library's own static workspace: allocates nothing (for callers that cannot allocate one).
inline void launch_mma_gemv_fp4_bf16_static(const uint16_t* act, size_t act_stride, const GlmFp4Matrix& w, uint16_t* out, int m,
                                            int n, int k, size_t out_stride, hipStream_t stream) {
  detail::check(dgpp_launch_mma_gemv_fp4_bf16_static(act, act_stride, &w, out, m, n, k, out_stride, stream));
}
inline void static_scratch_release() { detail::check(dgpp_static_scratch_release()); }
inline void launch_mma_gemv_fp4_f32(const uint16_t* act, size_t act_stride, const GlmFp4Matrix& w, float* out, int m, int n,
                                    int k, size_t out_stride, hipStream_t stream, void* ws = nullptr, size_t ws_bytes = 0) {
  detail::check(dgpp_launch_mma_gemv_fp4_f32(act, act_stride, &w, out, m, n, k, out_stride, stream, ws, ws_bytes));
}
inline void launch_mma_gemv_fp8_bf16(const uint16_t* act, size_t act_stride, const uint8_t* w, const float* scales,
                                     uint16_t* out, int m, int n, int k, size_t out_stride, int rs, int cs,
                                     hipStream_t stream, void* ws = nullptr, size_t ws_bytes = 0) {
  detail::check(dgpp_launch_mma_gemv_fp8_bf16(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws, ws_bytes));
}
inline void launch_mma_gemv_fp8_f32(const uint16_t* act, size_t act_stride, const uint8_t* w, const float* scales, float* out,
                                    int m, int n, int k, size_t out_stride, int rs, int cs, hipStream_t stream,
                                    void* ws = nullptr, size_t ws_bytes = 0) {
  detail::check(dgpp_launch_mma_gemv_fp8_f32(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws, ws_bytes));
}
inline void launch_mma_gemv_fp8e8m0_bf16(const uint16_t* act, size_t act_stride, const uint8_t* w, const uint8_t* scales,
                                         uint16_t* out, int m, int n, int k, size_t out_stride, int rs, int cs,
                                         hipStream_t stream, void* ws = nullptr, size_t ws_bytes = 0) {
  detail::check(dgpp_launch_mma_gemv_fp8e8m0_bf16(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws,
                                                  ws_bytes));
}
inline void launch_mma_gemv_fp8e8m0_f32(const uint16_t* act, size_t act_stride, const uint8_t* w, const uint8_t* scales,
                                        float* out, int m, int n, int k, size_t out_stride, int rs, int cs,
                                        hipStream_t stream, void* ws = nullptr, size_t ws_bytes = 0) {
  detail::check(dgpp_launch_mma_gemv_fp8e8m0_f32(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws,
                                                 ws_bytes));
}
inline void launch_moe_grouped_mma_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                        int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                        uint16_t* out, size_t out_stride, int n, int k, hipStream_t stream,
                                        const int32_t* act_rows = nullptr) {
  detail::check(dgpp_launch_moe_grouped_mma_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out,
                                                 out_stride, n, k, stream, act_rows));
}
inline void launch_moe_grouped_mma_f32(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                       int max_rows, int rows_per_block, const MoeExpertView* views, int which, float* out,
                                       size_t out_stride, int n, int k, hipStream_t stream,
                                       const int32_t* act_rows = nullptr) {
  detail::check(dgpp_launch_moe_grouped_mma_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out,
                                                out_stride, n, k, stream, act_rows));
}
// Timing-sweep knobs of the reference's kernels (src/kernels/glm_moe_launch.hpp:88-90, src/kernels/mma_gemv.hpp:132-135):
// accepted so that its benchmarks compile; this library's kernels have no counterpart setting and results never depended
// on them in the reference either.
inline void moe_set_fp8_ldm(bool) {}
inline void mma_gemv_set_decode_width(int) {}
inline bool mma_gemv_shape_ok(const void* w, const void* act, size_t act_stride, int m, int k) {
  return dgpp_mma_gemv_shape_ok(w, act, act_stride, m, k) != 0;
}
inline bool mma_gemv_pair_ok(const void* w0, const void* w1, const uint16_t* a0, const uint16_t* a1, size_t act_stride, int m,
                             int n0, int n1, int k, void* ws, size_t ws_bytes) {
  return dgpp_mma_gemv_pair_ok(w0, w1, a0, a1, act_stride, m, n0, n1, k, ws, ws_bytes) != 0;
}
inline void launch_mma_gemv_fp8_bf16_pair(const uint16_t* a0, const uint8_t* w0, const float* s0, uint16_t* o0, int n0,
                                          size_t stride0, const uint16_t* a1, const uint8_t* w1, const float* s1, uint16_t* o1,
                                          int n1, size_t stride1, size_t act_stride, int m, int k, int rs, int cs,
                                          hipStream_t stream, void* ws, size_t ws_bytes) {
  detail::check(dgpp_launch_mma_gemv_fp8_bf16_pair(a0, w0, s0, o0, n0, stride0, a1, w1, s1, o1, n1, stride1, act_stride, m, k, rs,
                                                   cs, stream, ws, ws_bytes));
}
inline void launch_mma_gemv_fp8_swiglu_f32(const uint16_t* gate, const uint16_t* up, float limit, size_t act_stride,
                                           const uint8_t* w, const float* scales, float* out, int m, int n, int k,
                                           size_t out_stride, int rs, int cs, hipStream_t stream) {
  detail::check(dgpp_launch_mma_gemv_fp8_swiglu_f32(gate, up, limit, act_stride, w, scales, out, m, n, k, out_stride, rs, cs,
                                                    stream));
}
// src/kernels/qwen_moe.hpp:18-87 (the shared gate and the FP8 forms of the shared expert's decode tail).
inline void qwen_moe_shared_gate_bf16(const uint16_t* x, const uint16_t* g, float* w, int tokens, int hidden, hipStream_t stream) {
  detail::check(dgpp_qwen_moe_shared_gate_bf16(x, g, w, tokens, hidden, stream));
}
inline void qwen_moe_shared_gate_up_decode_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                               const uint8_t* up_p, const float* up_s, const uint16_t* g, uint16_t* act,
                                               float* sw, int tokens, int H, int S, hipStream_t stream, int rs = 7, int cs = 7) {
  detail::check(dgpp_qwen_moe_shared_gate_up_decode_fp8(x, x_stride, gate_p, gate_s, up_p, up_s, g, act, sw, tokens, H, S, stream,
                                                        rs, cs));
}
inline void qwen_moe_shared_down_decode_fp8(const uint16_t* act, const uint8_t* down_p, const float* down_s, const float* sw,
                                            const float* acc, uint16_t* out, int tokens, int H, int S, hipStream_t stream,
                                            int rs = 7, int cs = 7) {
  detail::check(dgpp_qwen_moe_shared_down_decode_fp8(act, down_p, down_s, sw, acc, out, tokens, H, S, stream, rs, cs));
}
inline void qwen_moe_shared_down_decode_routed_fp8(const uint16_t* act, const uint8_t* down_p, const float* down_s,
                                                   const float* sw, const float* contrib, const float* weights, int top_k,
                                                   uint16_t* out, int tokens, int H, int S, hipStream_t stream, int rs = 7,
                                                   int cs = 7) {
  detail::check(dgpp_qwen_moe_shared_down_decode_routed_fp8(act, down_p, down_s, sw, contrib, weights, top_k, out, tokens, H, S,
                                                            stream, rs, cs));
}
inline void qwen_moe_shared_tail_decode_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                            const uint8_t* up_p, const float* up_s, const uint8_t* down_p, const float* down_s,
                                            const uint16_t* g, uint16_t* act, float* sw, const float* acc, uint16_t* out,
                                            int tokens, int H, int S, hipStream_t stream, int rs = 7, int cs = 7) {
  detail::check(dgpp_qwen_moe_shared_tail_decode_fp8(x, x_stride, gate_p, gate_s, up_p, up_s, down_p, down_s, g, act, sw, acc, out,
                                                     tokens, H, S, stream, rs, cs));
}
inline void qwen_moe_shared_tail_decode_routed_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                                   const uint8_t* up_p, const float* up_s, const uint8_t* down_p,
                                                   const float* down_s, const uint16_t* g, uint16_t* act, float* sw,
                                                   const float* contrib, const float* weights, int top_k, uint16_t* out,
                                                   int tokens, int H, int S, hipStream_t stream, int rs = 7, int cs = 7) {
  detail::check(dgpp_qwen_moe_shared_tail_decode_routed_fp8(x, x_stride, gate_p, gate_s, up_p, up_s, down_p, down_s, g, act, sw,
                                                            contrib, weights, top_k, out, tokens, H, S, stream, rs, cs));
}
// ---- activation-quantized NVFP4 (W4A4) form: src/kernels/moe_w4a4.hpp ----
inline size_t nvfp4_act_scale_stride(int k) { return dgpp_nvfp4_act_scale_stride(k); }
inline void launch_quantize_rows_nvfp4(const uint16_t* x, size_t x_stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                       float* gs, hipStream_t stream, float static_gs = 0.f,
                                       const float* static_gs_dev = nullptr) {
  detail::check(dgpp_launch_quantize_rows_nvfp4(x, x_stride, rows, k, codes, scales, gs, stream, static_gs, static_gs_dev));
}
inline void launch_swiglu_quantize_rows_nvfp4(const uint16_t* gate, const uint16_t* up, size_t stride, int rows, int k,
                                              float limit, uint8_t* codes, uint8_t* scales, float* gs, hipStream_t stream,
                                              float static_gs, const float* static_gs_dev = nullptr,
                                              bool qwen_rounding = false) {
  detail::check(dgpp_launch_swiglu_quantize_rows_nvfp4(gate, up, stride, rows, k, limit, codes, scales, gs, stream, static_gs,
                                                       static_gs_dev, qwen_rounding ? 1 : 0));
}
inline void launch_moe_grouped_w4a4_bf16(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                                         const MoeSegment* segs, int n_segs, int max_rows, const MoeExpertView* views,
                                         int which, uint16_t* out, size_t out_stride, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_grouped_w4a4_bf16(codes, scales, gs, act_rows, segs, n_segs, max_rows, views, which, out,
                                                  out_stride, n, k, stream));
}
inline void launch_moe_grouped_w4a4_f32(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                                        const MoeSegment* segs, int n_segs, int max_rows, const MoeExpertView* views,
                                        int which, float* out, size_t out_stride, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_moe_grouped_w4a4_f32(codes, scales, gs, act_rows, segs, n_segs, max_rows, views, which, out,
                                                 out_stride, n, k, stream));
}
// The dense form: the reference's TMA tensor maps become the code matrices' plain pointers (src/kernels/moe_w4a4.hpp:51-71).
inline bool dense_w4a4_supported(int k) { return dgpp_dense_w4a4_supported(k) != 0; }
inline void launch_dense_w4a4_bf16(const uint8_t* a_codes, const uint8_t* a_scales, size_t a_scale_stride, const float* a_gs,
                                   const uint8_t* w_codes, const uint8_t* w_scales, const float* w_global, uint16_t* out,
                                   size_t out_stride, int m, int n, int k, hipStream_t stream) {
  detail::check(dgpp_launch_dense_w4a4_bf16(a_codes, a_scales, a_scale_stride, a_gs, w_codes, w_scales, w_global, out, out_stride,
                                            m, n, k, stream));
}
// src/kernels/minimax_native_moe.hpp:8-18.
inline void minimax_quantize_rows_nvfp4(const uint16_t* input, size_t stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                        float* globals, hipStream_t stream) {
  detail::check(dgpp_minimax_quantize_rows_nvfp4(input, stride, rows, k, codes, scales, globals, stream));
}
inline void minimax_swiglu_f32(const float* gate, const float* up, uint16_t* output, int64_t count, float alpha, float limit,
                               hipStream_t stream) {
  detail::check(dgpp_minimax_swiglu_f32(gate, up, output, count, alpha, limit, stream));
}

// src/kernels/mxfp8_gemm.hpp:11-31.
inline void launch_mxfp8_quantize_rows(const uint16_t* x, size_t x_stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                       hipStream_t stream) {
  detail::check(dgpp_launch_mxfp8_quantize_rows(x, x_stride, rows, k, codes, scales, stream));
}
inline void launch_minimax_swiglu_mxfp8_rows(const uint16_t* gate, const uint16_t* up, size_t stride, int rows, int k,
                                             float alpha, float limit, uint8_t* codes, uint8_t* scales, hipStream_t stream) {
  detail::check(dgpp_launch_minimax_swiglu_mxfp8_rows(gate, up, stride, rows, k, alpha, limit, codes, scales, stream));
}
inline void launch_mxfp8_gemm_bf16(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales,
                                   uint16_t* out, int m, int n, int k, hipStream_t stream, size_t out_stride = 0,
                                   int output_tile = 0) {
  detail::check(dgpp_launch_mxfp8_gemm_bf16(a, a_scales, w, w_scales, out, m, n, k, stream, out_stride, output_tile));
}
inline void launch_mxfp8_gemm_f32(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales,
                                  float* out, int m, int n, int k, hipStream_t stream, size_t out_stride = 0,
                                  int output_tile = 0) {
  detail::check(dgpp_launch_mxfp8_gemm_f32(a, a_scales, w, w_scales, out, m, n, k, stream, out_stride, output_tile));
}
inline void launch_dense_mma_fp4_prod_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* seg,
                                           const MoeExpertView* views, int which, uint16_t* out, int m, int n, int k,
                                           hipStream_t stream, int fp4_group = kFp4Group) {
  detail::check(dgpp_launch_dense_mma_fp4_prod_bf16(act, act_stride, seg, views, which, out, m, n, k, stream, fp4_group));
}
inline bool dense_fp4_decode_shape(int m, int n, int k, int fp4_group = kFp4Group) {
  return dgpp_dense_fp4_decode_shape(m, n, k, fp4_group) != 0;
}
inline bool try_dense_fp4_decode_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* seg, const MoeExpertView* views,
                                      int which, uint16_t* out, int m, int n, int k, hipStream_t stream,
                                      int fp4_group = kFp4Group) {
  int launched = 0;
  detail::check(dgpp_try_dense_fp4_decode_bf16(act, act_stride, seg, views, which, out, m, n, k, stream, fp4_group, &launched));
  return launched != 0;
}
inline void launch_dense_mma_fp4_gate_up_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* seg,
                                              const MoeExpertView* views, uint16_t* gate, uint16_t* up, int m, int n, int k,
                                              hipStream_t stream, int fp4_group = kFp4Group) {
  detail::check(dgpp_launch_dense_mma_fp4_gate_up_bf16(act, act_stride, seg, views, gate, up, m, n, k, stream, fp4_group));
}
// Extension: grouped gate + up + SwiGLU in one matrix-core launch (see dgpp_amd.h).
inline void launch_moe_grouped_mma_gate_up_swiglu(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                                  int max_rows, int rows_per_block, const MoeExpertView* views,
                                                  uint16_t* out, size_t out_stride, int n, int k, float limit,
                                                  hipStream_t stream, const int32_t* act_rows = nullptr) {
  detail::check(dgpp_launch_moe_grouped_mma_gate_up_swiglu(act, act_stride, segs, n_segs, max_rows, rows_per_block, views,
                                                           out, out_stride, n, k, limit, stream, act_rows));
}
inline void launch_moe_grouped_mma_gate_up_swiglu_fp4(const uint16_t* act, size_t act_stride, const MoeSegment* segs,
                                                      int n_segs, int max_rows, int rows_per_block,
                                                      const MoeExpertView* views, uint16_t* out, size_t out_stride, int n,
                                                      int k, float limit, hipStream_t stream,
                                                      const int32_t* act_rows = nullptr, int fp4_group = kFp4Group) {
  detail::check(dgpp_launch_moe_grouped_mma_gate_up_swiglu_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views,
                                                               out, out_stride, n, k, limit, stream, act_rows, fp4_group));
}
inline void launch_moe_grouped_mma_fp4_bf16(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                            int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                            uint16_t* out, size_t out_stride, int n, int k, hipStream_t stream,
                                            const int32_t* act_rows = nullptr, int fp4_group = kFp4Group,
                                            int tile_rows = 64) {
  detail::check(dgpp_launch_moe_grouped_mma_fp4_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which,
                                                     out, out_stride, n, k, stream, act_rows, fp4_group, tile_rows));
}
inline void launch_moe_grouped_mma_fp4_f32(const uint16_t* act, size_t act_stride, const MoeSegment* segs, int n_segs,
                                           int max_rows, int rows_per_block, const MoeExpertView* views, int which,
                                           float* out, size_t out_stride, int n, int k, hipStream_t stream,
                                           const int32_t* act_rows = nullptr, int fp4_group = kFp4Group,
                                           int tile_rows = 64) {
  detail::check(dgpp_launch_moe_grouped_mma_fp4_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which,
                                                    out, out_stride, n, k, stream, act_rows, fp4_group, tile_rows));
}

// ---- src/kernels/scale_gemm.hpp ---------------------------------------------------------------------------
inline void launch_scale_gemm_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                   const float* w_scales, uint16_t* out, int m, int n, int k, hipStream_t stream,
                                   size_t out_row_stride_elems = 0, int mma_from_rows = 0, void* ws = nullptr,
                                   size_t ws_bytes = 0) {
  detail::check(dgpp_launch_scale_gemm_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                            out_row_stride_elems, mma_from_rows, ws, ws_bytes));
}
inline void launch_scale_gemm_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                  const float* w_scales, float* out, int m, int n, int k, hipStream_t stream,
                                  size_t out_row_stride_elems = 0, int mma_from_rows = 0, bool last_row_only = false,
                                  void* ws = nullptr, size_t ws_bytes = 0, int compact_row = -1) {
  detail::check(dgpp_launch_scale_gemm_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                           out_row_stride_elems, mma_from_rows, last_row_only ? 1 : 0, ws, ws_bytes,
                                           compact_row));
}
inline void launch_scale_gemm_grid_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                        const float* w_scales, uint16_t* out, int m, int n, int k, hipStream_t stream,
                                        size_t out_row_stride_elems, int rs, int cs, bool decode_mma = false,
                                        void* ws = nullptr, size_t ws_bytes = 0, bool prefill_tile = false) {
  detail::check(dgpp_launch_scale_gemm_grid_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                                 out_row_stride_elems, rs, cs, decode_mma, ws, ws_bytes, prefill_tile));
}
inline void launch_scale_gemm_grid_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                       const float* w_scales, float* out, int m, int n, int k, hipStream_t stream,
                                       size_t out_row_stride_elems, int rs, int cs, bool decode_mma = false,
                                       void* ws = nullptr, size_t ws_bytes = 0, bool prefill_tile = false) {
  detail::check(dgpp_launch_scale_gemm_grid_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                                out_row_stride_elems, rs, cs, decode_mma, ws, ws_bytes, prefill_tile));
}
inline void launch_scale_gemm_grid_e8m0_bf16(const uint16_t* act, size_t act_row_stride_elems,
                                             const uint8_t* w_payload, const uint8_t* w_scales, uint16_t* out, int m,
                                             int n, int k, hipStream_t stream, size_t out_row_stride_elems, int rs,
                                             int cs, void* ws = nullptr, size_t ws_bytes = 0,
                                             bool prefill_tile = false) {
  detail::check(dgpp_launch_scale_gemm_grid_e8m0_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k,
                                                      stream, out_row_stride_elems, rs, cs, ws, ws_bytes, prefill_tile));
}
inline void launch_scale_gemm_grid_e8m0_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                            const uint8_t* w_scales, float* out, int m, int n, int k,
                                            hipStream_t stream, size_t out_row_stride_elems, int rs, int cs,
                                            void* ws = nullptr, size_t ws_bytes = 0, bool prefill_tile = false) {
  detail::check(dgpp_launch_scale_gemm_grid_e8m0_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k,
                                                     stream, out_row_stride_elems, rs, cs, ws, ws_bytes, prefill_tile));
}
constexpr int kFp8GemvMaxProblems = 4;
inline void launch_scale_gemm_tile_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                        const float* w_scales, uint16_t* out, int m, int n, int k, hipStream_t stream,
                                        int rs = 7, int cs = 7) {
  detail::check(dgpp_launch_scale_gemm_tile_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream, rs, cs));
}
inline void launch_scale_gemm_tile_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                       const float* w_scales, float* out, int m, int n, int k, hipStream_t stream,
                                       int rs = 7, int cs = 7) {
  detail::check(dgpp_launch_scale_gemm_tile_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream, rs, cs));
}
inline void launch_scale_gemv_multi_bf16(const Fp8GemvProblem* problems, int n_problems, const uint16_t* act,
                                         size_t act_row_stride_elems, int rows, int k, hipStream_t stream) {
  detail::check(dgpp_launch_scale_gemv_multi_bf16(problems, n_problems, act, act_row_stride_elems, rows, k, stream));
}
inline bool fp8_gemv_can_stage(const void* w_payload, int k) { return dgpp_fp8_gemv_can_stage(w_payload, k) != 0; }

// ---- src/kernels/fp8_dequant.hpp ----------------------------------------------------------------------------
inline void launch_fp8_dequant_blocks(const uint8_t* payload, const float* scales, uint16_t* out_bf16, int64_t rows,
                                      int64_t cols, hipStream_t stream, int rs = 7, int cs = 7) {
  detail::check(dgpp_launch_fp8_dequant_blocks(payload, scales, out_bf16, rows, cols, stream, rs, cs));
}
inline void launch_fp8_dequant_blocks_e8m0(const uint8_t* payload, const uint8_t* scales, uint16_t* out_bf16,
                                           int64_t rows, int64_t cols, hipStream_t stream, int rs, int cs) {
  detail::check(dgpp_launch_fp8_dequant_blocks_e8m0(payload, scales, out_bf16, rows, cols, stream, rs, cs));
}

}  // namespace dgpp
