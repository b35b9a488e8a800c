// Host-side driver of one quantized MoE layer over the launcher surface (include/dgpp_amd.hpp):
// the counterpart of the reference's GlmMoeLayer (src/models/glm/moe_layer.hpp:50). It owns the
// layer's device scratch and device expert table, checks the weight geometry the way the
// reference's binding does (src/models/glm/moe_layer.cpp:527-583) and issues the reference's call
// order for the sync-free decode path (:1415-1680) and the device-segmented grouped path
// (:775-817, :906-934). All work is enqueued on the caller's stream; nothing synchronises.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <vector>

#include "../../include/dgpp_amd.hpp"

namespace dgpp {

enum class GlmExpertFormat { Fp8 = 0, Nvfp4 = 1, Mxfp4 = 2 };

struct GlmMoeLayerWeights {
  GlmExpertFormat format = GlmExpertFormat::Fp8;
  std::vector<MoeExpertView> views;   // [E * 3] (+3 when the shared expert is an FP4 table entry)
  bool shared_in_table = false;
  int shared_inter = 0;               // 0: no shared expert
  const uint8_t* sh_payload[3] = {nullptr, nullptr, nullptr};
  const float* sh_scales[3] = {nullptr, nullptr, nullptr};
  int sh_rs = 7, sh_cs = 7;
  // All three non-null: an MXFP8 shared expert (E8M0 byte per 32 columns) of its own width, run as dense projections.
  const uint8_t* sh_scales_e8m0[3] = {nullptr, nullptr, nullptr};
  const uint16_t* router_gate = nullptr;
  const float* router_bias = nullptr;
};

class GlmMoeLayer {
 public:
  GlmMoeLayer(const GlmMoeConfig& cfg, const GlmMoeLayerWeights& w, int max_tokens);
  ~GlmMoeLayer();
  GlmMoeLayer(const GlmMoeLayer&) = delete;
  GlmMoeLayer& operator=(const GlmMoeLayer&) = delete;

  static size_t scratch_bytes(const GlmMoeConfig& cfg, int max_tokens, int shared_inter, bool dense_shared = false);

  // out_f32 non-null: the unrounded chain goes there and out_bf16 is not written.
  void enqueue_decode(const uint16_t* x, size_t x_stride, uint16_t* out_bf16, float* out_f32, int tokens,
                      hipStream_t stream);
  // Synchronizes `stream` and throws std::runtime_error when a one-launch expert chain enqueued on it gave up its
  // bounded wait (its output is then invalid); the counters are back at rest afterwards.
  void check(hipStream_t stream);
  void enqueue_decode_scores(const uint16_t* x, size_t x_stride, const float* scores, const float* biased,
                             uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream);
  void enqueue_decode_routed(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                             uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream);
  void enqueue_grouped_routed(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                              uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream);
  // The same through the matrix-core grouped launchers (gather folded in, 16 token rows per weight pass); a layer's
  // shared expert rides along as the segment of every token (or as dense projections beside, the MXFP8 form).
  void enqueue_prefill_routed(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                              uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream);

  // The same from the hidden rows: score rows, selection, then the chain above over the layer's own routes.
  void enqueue_prefill(const uint16_t* x, size_t x_stride, uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream);
  // The prefill in phases over the layer's own routes: the router over rows [r0, r0 + rows), the chain over all rows
  // without its accumulation, the accumulation of rows [r0, r0 + rows) into out[r0 ...]. Bitwise enqueue_prefill.
  void route_prefill_rows(const uint16_t* x, size_t x_stride, int r0, int rows, hipStream_t stream);
  void enqueue_prefill_phased(const uint16_t* x, size_t x_stride, int tokens, hipStream_t stream);
  void accumulate_prefill_rows(uint16_t* out_bf16, float* out_f32, int tokens, int r0, int rows, hipStream_t stream);
  // The activation-quantized (W4A4) form of the same chain for NVFP4 experts: token rows and SwiGLU rows go through the
  // NVFP4 row quantizer. act_scales_dev: null (a global per row from the row's own maximum) or a DEVICE pair
  // {token rows' global, SwiGLU rows' global}. The down rows are bf16 unless f32_down or a shared expert's fp32 rows
  // sit behind them; the shared expert keeps BF16 activations (its segment, or dense projections beside).
  void enqueue_prefill_routed_w4a4(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                   uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream,
                                   const float* act_scales_dev = nullptr, bool f32_down = false);

  const MoeExpertView* views() const { return d_views_; }
  const int32_t* ids() const { return d_ids_; }
  const float* weights() const { return d_weights_; }
  bool has_shared() const { return w_.shared_inter > 0; }
  // The shared expert runs as dense projections over the token rows (MXFP8), not as slot top_k of every token.
  bool dense_shared() const { return has_shared() && w_.sh_scales_e8m0[0] != nullptr; }

 private:
  void release();
  void check_tokens(int tokens) const;
  bool needs_order(int tokens) const;
  void dense_shared_chain(const uint16_t* x, size_t x_stride, int tokens, hipStream_t stream);
  void prefill_chain(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights, uint16_t* out_bf16,
                     float* out_f32, int tokens, hipStream_t stream, bool with_shared, bool accumulate = true);
  void expert_chain_slots(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                          uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream,
                          bool order_ready = false, const float* sel_scores = nullptr, const float* sel_biased = nullptr,
                          bool routed_only = false);

  GlmMoeConfig cfg_;
  GlmMoeLayerWeights w_;
  int max_tokens_ = 0;
  int fp4_group_ = 16;
  int max_inter_ = 0;
  // One device allocation carved into the buffers below.
  void* arena_ = nullptr;
  MoeExpertView* d_views_ = nullptr;
  int32_t* d_ids_ = nullptr;
  float* d_weights_ = nullptr;
  float* d_scores_ = nullptr;
  float* d_biased_ = nullptr;
  int32_t* d_order_ = nullptr;
  uint16_t* d_slot_act_ = nullptr;   // [slots, max_inter]
  float* d_slot_down_ = nullptr;     // [slots, hidden]
  float* d_acc_ = nullptr;           // [tokens, hidden]
  int* d_tile_counter_ = nullptr;    // [2]
  int* d_chain_status_ = nullptr;    // raised by a one-launch chain whose bounded wait ran out
  uint32_t* d_chain_ready_ = nullptr;   // the one-launch chain's readiness words, zero at rest
  size_t counter_bytes_ = 0;
  // The shared expert's passes run beside the routed ones: a second stream of the default priority, forked from
  // and joined to the caller's stream with two events (created only for a layer with a shared expert).
  hipStream_t side_ = nullptr;
  hipEvent_t fork_ = nullptr, join_ = nullptr;
  int32_t* d_rows_ = nullptr;        // grouped path
  int32_t* d_slot_row_ = nullptr;
  MoeSegment* d_segs_ = nullptr;
  uint16_t* d_gather_ = nullptr;     // [rows_total, hidden]
  uint16_t* d_gate_ = nullptr;       // [rows_total, max_inter]
  uint16_t* d_up_ = nullptr;
  uint8_t* d_q_codes_ = nullptr;     // W4A4 operand rows: codes [slots, max(hidden, inter) / 2], scale bytes, globals
  uint8_t* d_q_scales_ = nullptr;
  float* d_q_gs_ = nullptr;
  MoeExpertView* d_sh_views_ = nullptr;   // [(n_experts + 1) * 3]: a block-FP8 shared expert as segment n_experts' entries
  // dense shared expert: gate / up / SwiGLU rows [tokens, shared_inter], unrounded down rows [tokens, hidden], the
  // split-K workspace of its projections, and the identity row list / unit weights of the last chain step
  uint16_t* d_sh_gate_ = nullptr;
  uint16_t* d_sh_up_ = nullptr;
  uint16_t* d_sh_act_ = nullptr;
  float* d_sh_down_ = nullptr;
  void* d_sh_ws_ = nullptr;
  size_t sh_ws_bytes_ = 0;
  int32_t* d_rows_id_ = nullptr;
  float* d_ones_ = nullptr;
};

}  // namespace dgpp
