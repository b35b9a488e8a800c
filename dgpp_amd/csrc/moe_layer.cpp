#include "moe_layer.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <stdexcept>
#include <string>

#include "../../include/dgpp_amd_bench.h"
#include "../../include/dgpp_amd_layer.h"

namespace dgpp {
namespace {

void hip_ok(hipError_t e, const char* what) {
  if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
size_t align_up(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

// Buffer sizes in bytes, in the order they are carved (each rounded to 256).
struct Layout {
  size_t views, ids, weights, scores, biased, order, slot_act, slot_down, acc, counter, rows, slot_row, segs, gather,
      gate, up, sh_gate, sh_up, sh_act, sh_down, sh_ws, rows_id, ones, q_codes, q_scales, q_gs, sh_views, total;
};
Layout layout_of(const GlmMoeConfig& c, int max_tokens, int shared_inter, size_t n_views, bool dense_shared) {
  const size_t M = static_cast<size_t>(std::max(max_tokens, 0)), H = c.hidden, K = c.top_k, E = c.n_experts;
  const size_t I = static_cast<size_t>(std::max(c.inter, shared_inter));
  const size_t slots = M * (K + 1);
  Layout l{};
  l.views = align_up(n_views * sizeof(MoeExpertView));
  l.ids = align_up(M * K * 4);
  l.weights = align_up(M * K * 4);
  l.scores = align_up(M * E * 4);
  l.biased = align_up(M * E * 4);
  l.order = align_up(slots * 4);
  l.slot_act = align_up(slots * I * 2);
  l.slot_down = align_up(slots * H * 4);
  l.acc = align_up(M * H * 4);
  // the stealing pair, the one-launch chain's status word (at +64 bytes) and its readiness words (from +256 bytes)
  l.counter = align_up(256 + M * K * 128);
  l.rows = align_up(slots * 4);
  l.slot_row = align_up(M * K * 4);
  l.segs = align_up((E + 1) * sizeof(MoeSegment));
  l.gather = align_up(slots * H * 2);
  l.gate = align_up(slots * I * 2);
  l.up = align_up(slots * I * 2);
  if (dense_shared) {
    const size_t SI = static_cast<size_t>(std::max(shared_inter, 0));
    l.sh_gate = l.sh_up = l.sh_act = align_up(M * SI * 2);
    l.sh_down = align_up(M * H * 4);
    l.sh_ws = align_up(4 * M * std::max(SI, H) * 4);   // up to four K parts of [tokens, n] partial sums
    l.rows_id = align_up(M * 4);
    l.ones = align_up(M * 4);
  }
  // The activation-quantized (W4A4) leg's operand rows: the token rows at K = hidden, then the slot rows at K = inter.
  const size_t qk = std::max(H, static_cast<size_t>(std::max(c.inter, 0)));
  l.q_codes = align_up(slots * (qk / 2));
  l.q_scales = align_up(slots * nvfp4_act_scale_stride(static_cast<int>(qk)));
  l.q_gs = align_up(slots * 4);
  // A block-FP8 shared expert handed over by pointers, as the table entries the grouped launchers read (its segment
  // names expert n_experts).
  l.sh_views = align_up((E + 1) * 3 * sizeof(MoeExpertView));
  l.total = l.views + l.ids + l.weights + l.scores + l.biased + l.order + l.slot_act + l.slot_down + l.acc + l.counter +
            l.rows + l.slot_row + l.segs + l.gather + l.gate + l.up + l.sh_gate + l.sh_up + l.sh_act + l.sh_down + l.sh_ws +
            l.rows_id + l.ones + l.q_codes + l.q_scales + l.q_gs + l.sh_views;
  return l;
}

// A branch of work on the side stream: forked from the caller's stream and joined to it again on EVERY way out of the
// scope that opened it (a launcher that throws between fork and join must not leave a captured graph with an
// unjoined branch).
struct StreamFork {
  hipStream_t main, side;
  hipEvent_t fork_ev, join_ev;
  bool open = false;
  void begin() {
    hip_ok(hipEventRecord(fork_ev, main), "GlmMoeLayer: fork");
    hip_ok(hipStreamWaitEvent(side, fork_ev, 0), "GlmMoeLayer: fork");
    open = true;
  }
  void end() {
    if (!open) return;
    open = false;
    hip_ok(hipEventRecord(join_ev, side), "GlmMoeLayer: join");
    hip_ok(hipStreamWaitEvent(main, join_ev, 0), "GlmMoeLayer: join");
  }
  ~StreamFork() {
    if (!open) return;
    if (hipEventRecord(join_ev, side) == hipSuccess) (void)hipStreamWaitEvent(main, join_ev, 0);
  }
};

}  // namespace

size_t GlmMoeLayer::scratch_bytes(const GlmMoeConfig& cfg, int max_tokens, int shared_inter, bool dense_shared) {
  return layout_of(cfg, max_tokens, shared_inter, static_cast<size_t>(cfg.n_experts + 1) * 3, dense_shared).total;
}

GlmMoeLayer::GlmMoeLayer(const GlmMoeConfig& cfg, const GlmMoeLayerWeights& w, int max_tokens)
    : cfg_(cfg), w_(w), max_tokens_(max_tokens) {
  GlmMoeConfig::validate_config(cfg);
  if (max_tokens <= 0) throw std::invalid_argument("GlmMoeLayer: max_tokens must be positive");
  const size_t E = static_cast<size_t>(cfg.n_experts);
  const bool fp4 = w.format != GlmExpertFormat::Fp8;
  fp4_group_ = w.format == GlmExpertFormat::Mxfp4 ? kMxfp4Group : kFp4Group;
  if (w.views.size() != (E + (w.shared_in_table ? 1 : 0)) * 3)
    throw std::runtime_error("GlmMoeLayer: the expert view table must hold n_experts (+1 shared) triples");
  // One format, one scale group and (FP8) one scale grid per matrix index across the table;
  // NVFP4 matrices carry a global (src/models/glm/moe_layer.cpp:527-583).
  auto grid_ok = [](int s) { return s >= 4 && s <= 7; };
  for (size_t i = 0; i < w.views.size(); ++i) {
    const MoeExpertView& v = w.views[i];
    if (!v.payload) throw std::runtime_error("GlmMoeLayer: inconsistent routed expert matrices (null payload)");
    if (fp4) {
      if (!v.fp4_scales || v.fp4_group != fp4_group_ || (fp4_group_ == kFp4Group && !v.fp4_global))
        throw std::runtime_error("GlmMoeLayer: inconsistent fp4 routed expert matrices (entry " + std::to_string(i) + ")");
    } else {
      const MoeExpertView& g = w.views[i % 3];
      if (!v.scales || v.scale_shift_rows != g.scale_shift_rows || v.scale_shift_cols != g.scale_shift_cols ||
          !grid_ok(v.scale_shift_rows) || !grid_ok(v.scale_shift_cols))
        throw std::runtime_error("GlmMoeLayer: inconsistent or unsupported expert scale grid (entry " +
                                 std::to_string(i) + ")");
    }
  }
  const bool e8m0_shared = w.sh_scales_e8m0[0] || w.sh_scales_e8m0[1] || w.sh_scales_e8m0[2];
  if (e8m0_shared) {
    if (w.shared_in_table || w.shared_inter <= 0)
      throw std::runtime_error("GlmMoeLayer: an MXFP8 shared expert is given by payloads and scale bytes and needs its width");
    for (int i = 0; i < 3; ++i)
      if (!w.sh_payload[i] || !w.sh_scales_e8m0[i]) throw std::runtime_error("GlmMoeLayer: inconsistent MXFP8 shared matrices");
    if (cfg.hidden % 32 != 0 || w.shared_inter % 32 != 0)
      throw std::runtime_error("GlmMoeLayer: an MXFP8 shared expert needs hidden and its width in multiples of 32");
  } else if (w.shared_in_table) {
    if (!fp4) throw std::runtime_error("GlmMoeLayer: a table-resident shared expert needs an fp4 table");
    if (w.shared_inter != cfg.inter)
      throw std::runtime_error(
          "GlmMoeLayer: the NVFP4 shared expert's inter must equal the routed experts' (the slot kernels' K)");
  } else if (w.shared_inter > 0) {
    for (int i = 0; i < 3; ++i)
      if (!w.sh_payload[i] || !w.sh_scales[i]) throw std::runtime_error("GlmMoeLayer: inconsistent shared matrices");
  }
  if ((cfg.n_shared_experts != 0) != (w.shared_inter > 0))
    throw std::runtime_error("GlmMoeLayer: n_shared_experts does not match the shared weights");
  max_inter_ = e8m0_shared ? cfg.inter : std::max(cfg.inter, w.shared_inter);   // a dense shared expert takes no slot rows

  const Layout l = layout_of(cfg, max_tokens, w.shared_inter, w.views.size(), e8m0_shared);
  hip_ok(hipMalloc(&arena_, l.total), "GlmMoeLayer: hipMalloc");
  try {
  uint8_t* p = static_cast<uint8_t*>(arena_);
  auto carve = [&p](size_t bytes) {
    uint8_t* q = p;
    p += bytes;
    return q;
  };
  d_views_ = reinterpret_cast<MoeExpertView*>(carve(l.views));
  d_ids_ = reinterpret_cast<int32_t*>(carve(l.ids));
  d_weights_ = reinterpret_cast<float*>(carve(l.weights));
  d_scores_ = reinterpret_cast<float*>(carve(l.scores));
  d_biased_ = reinterpret_cast<float*>(carve(l.biased));
  d_order_ = reinterpret_cast<int32_t*>(carve(l.order));
  d_slot_act_ = reinterpret_cast<uint16_t*>(carve(l.slot_act));
  d_slot_down_ = reinterpret_cast<float*>(carve(l.slot_down));
  d_acc_ = reinterpret_cast<float*>(carve(l.acc));
  d_tile_counter_ = reinterpret_cast<int*>(carve(l.counter));
  d_chain_status_ = d_tile_counter_ + 16;
  d_chain_ready_ = reinterpret_cast<uint32_t*>(d_tile_counter_ + 64);
  counter_bytes_ = l.counter;
  d_rows_ = reinterpret_cast<int32_t*>(carve(l.rows));
  d_slot_row_ = reinterpret_cast<int32_t*>(carve(l.slot_row));
  d_segs_ = reinterpret_cast<MoeSegment*>(carve(l.segs));
  d_gather_ = reinterpret_cast<uint16_t*>(carve(l.gather));
  d_gate_ = reinterpret_cast<uint16_t*>(carve(l.gate));
  d_up_ = reinterpret_cast<uint16_t*>(carve(l.up));
  if (e8m0_shared) {
    d_sh_gate_ = reinterpret_cast<uint16_t*>(carve(l.sh_gate));
    d_sh_up_ = reinterpret_cast<uint16_t*>(carve(l.sh_up));
    d_sh_act_ = reinterpret_cast<uint16_t*>(carve(l.sh_act));
    d_sh_down_ = reinterpret_cast<float*>(carve(l.sh_down));
    d_sh_ws_ = carve(l.sh_ws);
    sh_ws_bytes_ = l.sh_ws;
    d_rows_id_ = reinterpret_cast<int32_t*>(carve(l.rows_id));
    d_ones_ = reinterpret_cast<float*>(carve(l.ones));
    std::vector<int32_t> idv(static_cast<size_t>(max_tokens));
    std::vector<float> onev(static_cast<size_t>(max_tokens), 1.0f);
    for (int i = 0; i < max_tokens; ++i) idv[static_cast<size_t>(i)] = i;
    hip_ok(hipMemcpy(d_rows_id_, idv.data(), idv.size() * 4, hipMemcpyHostToDevice), "GlmMoeLayer: row list upload");
    hip_ok(hipMemcpy(d_ones_, onev.data(), onev.size() * 4, hipMemcpyHostToDevice), "GlmMoeLayer: unit weights upload");
  }
  d_q_codes_ = carve(l.q_codes);
  d_q_scales_ = carve(l.q_scales);
  d_q_gs_ = reinterpret_cast<float*>(carve(l.q_gs));
  d_sh_views_ = reinterpret_cast<MoeExpertView*>(carve(l.sh_views));
  if (w.shared_inter > 0 && !w.shared_in_table && !e8m0_shared) {
    std::vector<MoeExpertView> table((E + 1) * 3);
    for (int i = 0; i < 3; ++i) {
      MoeExpertView& v = table[E * 3 + static_cast<size_t>(i)];
      v.payload = w.sh_payload[i];
      v.scales = w.sh_scales[i];
      v.scale_shift_rows = w.sh_rs;
      v.scale_shift_cols = w.sh_cs;
      v.fp4_group = kFp4Group;
    }
    hip_ok(hipMemcpy(d_sh_views_, table.data(), table.size() * sizeof(MoeExpertView), hipMemcpyHostToDevice),
           "GlmMoeLayer: shared table upload");
  }
  // The device expert table is uploaded once (the reference's capture form prepares a per-binding
  // device table once too, src/models/glm/moe_layer.cpp:364-396); the counter pair is zero at rest.
  hip_ok(hipMemcpy(d_views_, w.views.data(), w.views.size() * sizeof(MoeExpertView), hipMemcpyHostToDevice),
         "GlmMoeLayer: table upload");
  hip_ok(hipMemset(d_tile_counter_, 0, counter_bytes_), "GlmMoeLayer: counters");
  if (has_shared()) {
    hip_ok(hipStreamCreateWithFlags(&side_, hipStreamNonBlocking), "GlmMoeLayer: side stream");
    hip_ok(hipEventCreateWithFlags(&fork_, hipEventDisableTiming), "GlmMoeLayer: event");
    hip_ok(hipEventCreateWithFlags(&join_, hipEventDisableTiming), "GlmMoeLayer: event");
  }
  } catch (...) {   // a throwing constructor runs no destructor: give back what was taken so far
    release();
    throw;
  }
}

void GlmMoeLayer::release() {
  if (join_) (void)hipEventDestroy(join_);
  if (fork_) (void)hipEventDestroy(fork_);
  if (side_) (void)hipStreamDestroy(side_);
  if (arena_) (void)hipFree(arena_);
  join_ = fork_ = nullptr;
  side_ = nullptr;
  arena_ = nullptr;
}

GlmMoeLayer::~GlmMoeLayer() { release(); }

// The expert-sorted slot order pays for itself once many slots share experts. A small batch (tokens * top_k <=
// 64) skips it: the gate/up kernel finds the few sharers by ballot, the token-major down kernel needs no order,
// and the selection runs as one wavefront per token on separate CUs instead of one block.
bool GlmMoeLayer::needs_order(int tokens) const {
  if (tokens <= 1 || tokens * (cfg_.top_k + 1) > 1024) return false;
  if (dgpp_tune_get(6) == 1) return true;
  return tokens * cfg_.top_k > 128;   // up to 128 routed slots the gate/up kernel finds the sharers of an expert by ballot
}

// Waits for `stream` and reads the one-launch chain's status word: a launch whose bounded wait ran out has
// produced nothing valid. The counters are put back to rest before the error is raised.
void GlmMoeLayer::check(hipStream_t stream) {
  hip_ok(hipStreamSynchronize(stream), "GlmMoeLayer: check");
  int status = 0;
  hip_ok(hipMemcpy(&status, d_chain_status_, sizeof(int), hipMemcpyDeviceToHost), "GlmMoeLayer: check");
  if (status == 0) return;
  hip_ok(hipMemset(d_tile_counter_, 0, counter_bytes_), "GlmMoeLayer: counters");
  throw std::runtime_error("GlmMoeLayer: a one-launch expert chain gave up waiting for its gate/up rows; the output of "
                           "that call is invalid");
}

void GlmMoeLayer::check_tokens(int tokens) const {
  if (tokens > max_tokens_) throw std::invalid_argument("GlmMoeLayer: tokens exceed the layer's max_tokens");
}

void GlmMoeLayer::enqueue_decode(const uint16_t* x, size_t x_stride, uint16_t* out_bf16, float* out_f32, int tokens,
                                 hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  if (!w_.router_gate) throw std::invalid_argument("GlmMoeLayer: the router gate is not bound");
  // The score rows, then the chain from given scores: the selection rides a later launch where one takes it
  // (with the slot order, or inside the gate/up launch of a one-token step).
  launch_moe_router_dots(x, w_.router_gate, w_.router_bias, d_scores_, d_biased_, cfg_, tokens, stream);
  enqueue_decode_scores(x, x_stride, d_scores_, d_biased_, out_bf16, out_f32, tokens, stream);
}

void GlmMoeLayer::enqueue_decode_scores(const uint16_t* x, size_t x_stride, const float* scores, const float* biased,
                                        uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  // One routed-only token: the gate/up launch repeats the selection in its blocks (no launch of its own).
  // Otherwise selection and slot order in one launch; the chain below then finds its order ready.
  const bool with_order = needs_order(tokens);
  const bool fused = tokens == 1 && dgpp_tune_get(7) != 1;
  if (!fused)
    launch_moe_router_select_order(scores, biased, d_ids_, d_weights_, with_order ? d_order_ : nullptr, cfg_, tokens, stream,
                                   cfg_.shared_slots_early);
  expert_chain_slots(x, x_stride, d_ids_, d_weights_, out_bf16, out_f32, tokens, stream, /*order_ready=*/true,
                     fused ? scores : nullptr, fused ? biased : nullptr);
}

void GlmMoeLayer::enqueue_decode_routed(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                        uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  expert_chain_slots(x, x_stride, ids, weights, out_bf16, out_f32, tokens, stream);
}

// The dense shared expert: gate and up projections of every token row, SwiGLU, the down projection (unrounded).
void GlmMoeLayer::dense_shared_chain(const uint16_t* x, size_t x_stride, int tokens, hipStream_t st) {
  const int H = cfg_.hidden, SI = w_.shared_inter;
  launch_scale_gemm_grid_e8m0_bf16(x, x_stride, w_.sh_payload[0], w_.sh_scales_e8m0[0], d_sh_gate_, tokens, SI, H, st,
                                   static_cast<size_t>(SI), 0, 5, d_sh_ws_, sh_ws_bytes_);
  launch_scale_gemm_grid_e8m0_bf16(x, x_stride, w_.sh_payload[1], w_.sh_scales_e8m0[1], d_sh_up_, tokens, SI, H, st,
                                   static_cast<size_t>(SI), 0, 5, d_sh_ws_, sh_ws_bytes_);
  launch_moe_swiglu_clamp(d_sh_gate_, d_sh_up_, d_sh_act_, static_cast<int64_t>(tokens) * SI, cfg_.swiglu_limit, st);
  launch_scale_gemm_grid_e8m0_f32(d_sh_act_, static_cast<size_t>(SI), w_.sh_payload[2], w_.sh_scales_e8m0[2], d_sh_down_,
                                  tokens, H, SI, st, static_cast<size_t>(H), 0, 5, d_sh_ws_, sh_ws_bytes_);
}

// Steps 4-7 of the reference's decode call order (src/models/glm/moe_layer.cpp:1555-1677).
void GlmMoeLayer::expert_chain_slots(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                     uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream,
                                     bool order_ready, const float* sel_scores, const float* sel_biased,
                                     bool routed_only) {
  const int K = cfg_.top_k, H = cfg_.hidden, I = cfg_.inter;
  if (out_bf16 == nullptr && out_f32 == nullptr) throw std::invalid_argument("GlmMoeLayer: no output buffer");
  if (dense_shared() && !routed_only) {
    // The routed chain, unrounded, with the shared expert's dense projections beside it on the side stream (they
    // depend on nothing but x); then the chain's last step a = fma(1, shared, a) and the one rounding.
    float* acc = out_f32 ? out_f32 : d_acc_;
    StreamFork fork{stream, side_, fork_, join_};
    const bool beside = side_ != nullptr && dgpp_tune_get(9) != 1;
    if (beside) {
      fork.begin();
      dense_shared_chain(x, x_stride, tokens, side_);
    }
    expert_chain_slots(x, x_stride, ids, weights, nullptr, acc, tokens, stream, order_ready, sel_scores, sel_biased,
                       /*routed_only=*/true);
    if (beside) fork.end();
    else dense_shared_chain(x, x_stride, tokens, stream);
    launch_moe_accum(acc, d_sh_down_, d_rows_id_, d_ones_, tokens, H, stream);
    if (!out_f32) launch_moe_round_bf16(out_bf16, acc, static_cast<int64_t>(tokens) * H, stream);
    return;
  }
  const bool slot_shared = has_shared() && !dense_shared();   // the shared expert as slot top_k of every token
  const int slots = tokens * (K + 1);
  if (slots > 1024 && tokens > 1)
    throw std::invalid_argument("GlmMoeLayer: the decode-slot path takes at most 1024 slots; use the grouped path");
  const int32_t* order = nullptr;
  if (needs_order(tokens)) {
    if (!order_ready) launch_moe_slot_order(ids, d_order_, slots, K, cfg_.n_experts, stream, cfg_.shared_slots_early);
    order = d_order_;
  }
  // The token-major down kernel fuses the accumulation but reads an expert once per slot; the slot kernel reads
  // it once per run of slots. Token-major while few slots can share an expert (small batches), runs beyond.
  const bool token_major = !slot_shared && dgpp_tune_get(4) != 1 && tokens * K * 2 <= cfg_.n_experts;
  const bool sh_args = slot_shared && !w_.shared_in_table;
  const int n_sh = slot_shared ? w_.shared_inter : 0;
  const int k_sh_up = slot_shared ? H : 0;     // the shared gate/up contract over hidden
  // With scores given, ids / weights are this layer's own buffers and the gate/up launch fills them.
  const bool fused = sel_scores != nullptr && ids == d_ids_ && weights == d_weights_ && order == nullptr;
  if (sel_scores != nullptr && !fused) throw std::logic_error("GlmMoeLayer: fused selection outside its form");
  // The shared expert's gate/up and down passes read nothing the routed passes write (disjoint slot rows): they run
  // on the side stream beside them, forked here and joined before the accumulation. One launcher call per pass.
  // From a few tokens on: the two cross-stream dependencies cost more than the two hand-overs they take off the
  // chain while a pass is only a few microseconds long (measured: slower at one token, level at two).
  const bool split = slot_shared && side_ != nullptr && dgpp_tune_get(9) != 1 && (tokens >= 3 || dgpp_tune_get(9) == 2);
  // On one stream the shared down pass ends with the token's accumulation (no launch of its own).
  // (One token, where a launch is a fifth of the step; measured level at two tokens. Bench switch 9 = 4 folds at any
  // batch size, 3 never.)
  const bool fold_accum = slot_shared && !split && out_bf16 != nullptr && out_f32 == nullptr && dgpp_tune_get(9) != 3 &&
                          (tokens == 1 || dgpp_tune_get(9) == 4);
  // Everything that can be refused is refused before the first enqueue.
  if (slot_shared && out_f32 != nullptr)
    throw std::invalid_argument("GlmMoeLayer: an unrounded output with a shared expert is not a decode form");
  if (out_bf16 == nullptr && out_f32 == nullptr) throw std::invalid_argument("GlmMoeLayer: no output buffer");
  StreamFork fork{stream, side_, fork_, join_};
  if (split) fork.begin();
  // One launcher call per pass and stream: the routed pass on the caller's stream, the shared pass beside it.
  auto for_passes = [&](auto&& call) {
    if (!split) return call(stream, 3);
    call(stream, 1);
    call(side_, 2);
  };
  const float* fold_w = fold_accum ? weights : nullptr;
  uint16_t* fold_o = fold_accum ? out_bf16 : nullptr;
  // Routed only, a small batch: gate/up, down and the accumulation in ONE launch (dgpp_launch_moe_slot_chain*), with
  // the selection of a one-token step inside it. Measured slower than the launches it stands for on this chip at
  // every batch size (one register budget for both parts, and the readers' polls of the readiness words), so the
  // driver takes it only under bench switch 12 = 2.
  const bool one_launch = token_major && !fused && dgpp_tune_get(12) == 2;
  const bool one_launch_sel = token_major && fused && dgpp_tune_get(12) == 2;
  if (w_.format == GlmExpertFormat::Fp8) {
    if (one_launch_sel) {
      launch_moe_select_slot_chain(sel_scores, sel_biased, d_ids_, d_weights_, cfg_, tokens, x, x_stride, d_views_, I, H,
                                   d_slot_act_, max_inter_, cfg_.swiglu_limit, out_bf16, out_f32, d_chain_ready_,
                                   d_chain_status_, stream);
      return;
    }
    if (one_launch) {
      launch_moe_slot_chain(x, x_stride, ids, d_views_, I, H, d_slot_act_, max_inter_, tokens, K, cfg_.swiglu_limit, weights,
                            out_bf16, out_f32, d_chain_ready_, d_chain_status_, stream);
      return;
    }
    if (fused) {
      launch_moe_select_gate_up_swiglu(sel_scores, sel_biased, d_ids_, d_weights_, cfg_, tokens, x, x_stride, d_views_, I, H,
                                       d_slot_act_, max_inter_, cfg_.swiglu_limit, stream);
      if (slot_shared)   // the shared slot's pass: the routed pass already ran above
        launch_moe_slot_gate_up_swiglu_ex(x, x_stride, ids, order, d_views_, I, H, n_sh, k_sh_up, w_.sh_payload[0],
                                          w_.sh_scales[0], w_.sh_payload[1], w_.sh_scales[1], d_slot_act_, max_inter_, slots,
                                          K, cfg_.swiglu_limit, split ? side_ : stream, w_.sh_rs, w_.sh_cs, 2);
    } else
      for_passes([&](hipStream_t st, int passes) {
        launch_moe_slot_gate_up_swiglu_ex(x, x_stride, ids, order, d_views_, I, H, n_sh, k_sh_up, w_.sh_payload[0],
                                          w_.sh_scales[0], w_.sh_payload[1], w_.sh_scales[1], d_slot_act_, max_inter_, slots,
                                          K, cfg_.swiglu_limit, st, w_.sh_rs, w_.sh_cs, passes);
      });
    if (token_major) {   // routed only: down + accumulation in one token-major launch
      launch_moe_slot_down_accum(d_slot_act_, static_cast<size_t>(max_inter_), ids, d_views_, H, I, tokens, K, weights,
                                 out_bf16, out_f32, stream);
      return;
    }
    for_passes([&](hipStream_t st, int passes) {
      launch_moe_slot_down_ex(d_slot_act_, static_cast<size_t>(max_inter_), ids, order, d_views_, H, I, slot_shared ? H : 0,
                              n_sh, w_.sh_payload[2], w_.sh_scales[2], d_slot_down_, H, slots, K, st, w_.sh_rs, w_.sh_cs,
                              passes, fold_w, fold_o);
    });
  } else {
    const int base = w_.shared_in_table ? cfg_.n_experts * 3 : -1;
    if (one_launch_sel) {
      launch_moe_select_slot_chain_fp4(sel_scores, sel_biased, d_ids_, d_weights_, cfg_, tokens, x, x_stride, d_views_, I, H,
                                       d_slot_act_, max_inter_, cfg_.swiglu_limit, out_bf16, out_f32, d_chain_ready_,
                                       d_chain_status_, stream, fp4_group_);
      return;
    }
    if (one_launch) {
      launch_moe_slot_chain_fp4(x, x_stride, ids, d_views_, I, H, d_slot_act_, max_inter_, tokens, K, cfg_.swiglu_limit,
                                weights, out_bf16, out_f32, d_chain_ready_, d_chain_status_, stream, fp4_group_);
      return;
    }
    if (fused) {
      launch_moe_select_gate_up_swiglu_fp4(sel_scores, sel_biased, d_ids_, d_weights_, cfg_, tokens, x, x_stride, d_views_, I,
                                           H, d_slot_act_, max_inter_, cfg_.swiglu_limit, stream, fp4_group_);
      if (slot_shared)
        launch_moe_slot_gate_up_swiglu_fp4_ex(x, x_stride, ids, order, d_views_, I, H, n_sh, k_sh_up,
                                              sh_args ? w_.sh_payload[0] : nullptr, sh_args ? w_.sh_scales[0] : nullptr,
                                              sh_args ? w_.sh_payload[1] : nullptr, sh_args ? w_.sh_scales[1] : nullptr,
                                              d_slot_act_, max_inter_, slots, K, cfg_.swiglu_limit, split ? side_ : stream,
                                              base, fp4_group_, w_.sh_rs, w_.sh_cs, 2);
    } else
      for_passes([&](hipStream_t st, int passes) {
        launch_moe_slot_gate_up_swiglu_fp4_ex(x, x_stride, ids, order, d_views_, I, H, n_sh, k_sh_up,
                                              sh_args ? w_.sh_payload[0] : nullptr, sh_args ? w_.sh_scales[0] : nullptr,
                                              sh_args ? w_.sh_payload[1] : nullptr, sh_args ? w_.sh_scales[1] : nullptr,
                                              d_slot_act_, max_inter_, slots, K, cfg_.swiglu_limit, st, base, fp4_group_,
                                              w_.sh_rs, w_.sh_cs, passes);
      });
    if (token_major) {
      launch_moe_slot_down_accum_fp4(d_slot_act_, static_cast<size_t>(max_inter_), ids, d_views_, H, I, tokens, K, weights,
                                     out_bf16, out_f32, stream, fp4_group_);
      return;
    }
    for_passes([&](hipStream_t st, int passes) {
      launch_moe_slot_down_fp4_ex(d_slot_act_, static_cast<size_t>(max_inter_), ids, order, d_views_, H, I,
                                  slot_shared ? H : 0, n_sh, sh_args ? w_.sh_payload[2] : nullptr,
                                  sh_args ? w_.sh_scales[2] : nullptr, d_slot_down_, H, slots, K, st, base, fp4_group_,
                                  w_.sh_rs, w_.sh_cs, d_tile_counter_, passes, fold_w, fold_o);
    });
  }
  fork.end();
  if (fold_accum) return;
  if (slot_shared) {
    launch_moe_slot_accum(out_bf16, d_slot_down_, weights, tokens, H, K, stream);
  } else if (out_f32) {
    launch_moe_slot_accum_routed_f32(out_f32, d_slot_down_, weights, tokens, H, K, stream);
  } else {
    launch_moe_slot_accum_routed_bf16(out_bf16, d_slot_down_, weights, tokens, H, K, stream);
  }
}

// The device-segmented grouped path (src/models/glm/moe_layer.cpp:906-934, :1054-1379 GEMV form).
void GlmMoeLayer::enqueue_grouped_routed(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                         uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  if (has_shared())
    throw std::invalid_argument("GlmMoeLayer: the grouped path here covers the routed experts (no shared segment)");
  if (x_stride != static_cast<size_t>(cfg_.hidden))
    throw std::invalid_argument("GlmMoeLayer: the grouped path gathers dense [tokens, hidden] rows");
  const int K = cfg_.top_k, H = cfg_.hidden, I = cfg_.inter, E = cfg_.n_experts;
  const int tk = tokens * K;
  launch_moe_segment(ids, tokens, K, E, d_rows_, d_slot_row_, d_segs_, stream);
  launch_moe_gather_rows(x, d_rows_, d_gather_, tk, H, stream);
  const int max_rows = tokens;  // a segment holds at most one row per token
  if (w_.format == GlmExpertFormat::Fp8) {
    launch_moe_grouped_gemv_bf16(d_gather_, H, d_segs_, E, max_rows, 0, d_views_, 0, d_gate_, I, I, H, stream);
    launch_moe_grouped_gemv_bf16(d_gather_, H, d_segs_, E, max_rows, 0, d_views_, 1, d_up_, I, I, H, stream);
  } else {
    launch_moe_grouped_gemv_fp4_bf16(d_gather_, H, d_segs_, E, max_rows, 0, d_views_, 0, d_gate_, I, I, H, stream,
                                     fp4_group_);
    launch_moe_grouped_gemv_fp4_bf16(d_gather_, H, d_segs_, E, max_rows, 0, d_views_, 1, d_up_, I, I, H, stream,
                                     fp4_group_);
  }
  launch_moe_swiglu_clamp(d_gate_, d_up_, d_slot_act_, static_cast<int64_t>(tk) * I, cfg_.swiglu_limit, stream);
  if (w_.format == GlmExpertFormat::Fp8)
    launch_moe_grouped_gemv_f32(d_slot_act_, I, d_segs_, E, max_rows, 0, d_views_, 2, d_slot_down_, H, H, I, stream);
  else
    launch_moe_grouped_gemv_fp4_f32(d_slot_act_, I, d_segs_, E, max_rows, 0, d_views_, 2, d_slot_down_, H, H, I, stream,
                                    fp4_group_);
  if (out_f32)
    launch_moe_accum_ordered_f32(out_f32, d_slot_down_, H, d_slot_row_, ids, weights, -1, tokens, K, H, stream);
  else
    launch_moe_accum_ordered(out_bf16, d_slot_down_, H, d_slot_row_, ids, weights, -1, tokens, K, H, stream);
}

// The matrix-core grouped path (the reference's prefill form, src/models/glm/moe_layer.cpp:775-817): the same
// stages as enqueue_grouped_routed with the gather folded into the gate / up launches (act_rows) and 16 token
// rows per weight pass.
void GlmMoeLayer::enqueue_prefill_routed(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                         uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  if (out_bf16 == nullptr && out_f32 == nullptr) throw std::invalid_argument("GlmMoeLayer: no output buffer");
  if (dense_shared()) {
    const int H = cfg_.hidden;
    // As in the decode chain: the routed rows unrounded, the shared expert's dense projections beside them on the
    // side stream, then a = fma(1, shared, a) and the one rounding.
    float* acc = out_f32 ? out_f32 : d_acc_;
    StreamFork fork{stream, side_, fork_, join_};
    fork.begin();
    dense_shared_chain(x, x_stride, tokens, side_);
    prefill_chain(x, x_stride, ids, weights, nullptr, acc, tokens, stream, /*with_shared=*/false);
    fork.end();
    launch_moe_accum(acc, d_sh_down_, d_rows_id_, d_ones_, tokens, H, stream);
    if (!out_f32) launch_moe_round_bf16(out_bf16, acc, static_cast<int64_t>(tokens) * H, stream);
    return;
  }
  prefill_chain(x, x_stride, ids, weights, out_bf16, out_f32, tokens, stream, has_shared());
}

// The whole prefill step from the hidden rows (reference: GlmMoeLayer::enqueue_prefill, src/models/glm/moe_layer.cpp:775-812
// - route on the device, then the grouped chain, nothing waits on the host): score rows, selection, enqueue_prefill_routed
// over the layer's own ids and weights.
void GlmMoeLayer::enqueue_prefill(const uint16_t* x, size_t x_stride, uint16_t* out_bf16, float* out_f32, int tokens,
                                  hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  if (!w_.router_gate) throw std::invalid_argument("GlmMoeLayer: the router gate is not bound");
  launch_moe_router_dots(x, w_.router_gate, w_.router_bias, d_scores_, d_biased_, cfg_, tokens, stream);
  launch_moe_router_select(d_scores_, d_biased_, d_ids_, d_weights_, cfg_, tokens, stream);
  enqueue_prefill_routed(x, x_stride, d_ids_, d_weights_, out_bf16, out_f32, tokens, stream);
}

// Segments -> gate + up + SwiGLU -> down -> ordered accumulation on the matrix core. with_shared: the shared expert
// is segment n_experts (every token, in token order, rows [tokens * top_k, ...) of the slot buffers; the reference's
// shared_seg, src/models/glm/moe_layer.cpp:1293-1296, 1335-1336) and ends every token's chain with weight 1.
void GlmMoeLayer::prefill_chain(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream, bool with_shared,
                                bool accumulate) {
  const int K = cfg_.top_k, H = cfg_.hidden, I = cfg_.inter, E = cfg_.n_experts;
  const int tk = tokens * K;
  const bool fp8 = w_.format == GlmExpertFormat::Fp8;
  const bool in_table = with_shared && w_.shared_in_table;   // the routed experts' format and width: one more segment
  const size_t stride = with_shared ? static_cast<size_t>(max_inter_) : static_cast<size_t>(I);
  const int n_segs = in_table ? E + 1 : E;
  launch_moe_segment(ids, tokens, K, E, d_rows_, d_slot_row_, d_segs_, stream);
  const int max_rows = tokens;
  // gate + up + SwiGLU in one launch (the bits of the two grouped launches and the elementwise kernel)
  if (fp8)
    launch_moe_grouped_mma_gate_up_swiglu(x, x_stride, d_segs_, n_segs, max_rows, 0, d_views_, d_slot_act_, stride, I, H,
                                          cfg_.swiglu_limit, stream, d_rows_);
  else
    launch_moe_grouped_mma_gate_up_swiglu_fp4(x, x_stride, d_segs_, n_segs, max_rows, 0, d_views_, d_slot_act_, stride, I, H,
                                              cfg_.swiglu_limit, stream, d_rows_, fp4_group_);
  if (with_shared && !in_table)   // a block-FP8 shared expert of its own width
    launch_moe_grouped_mma_gate_up_swiglu(x, x_stride, d_segs_ + E, 1, max_rows, 0, d_sh_views_, d_slot_act_, stride,
                                          w_.shared_inter, H, cfg_.swiglu_limit, stream, d_rows_);
  if (fp8)
    launch_moe_grouped_mma_f32(d_slot_act_, stride, d_segs_, n_segs, max_rows, 0, d_views_, 2, d_slot_down_, H, H, I, stream);
  else
    launch_moe_grouped_mma_fp4_f32(d_slot_act_, stride, d_segs_, n_segs, max_rows, 0, d_views_, 2, d_slot_down_, H, H, I, stream,
                                   nullptr, fp4_group_);
  if (with_shared && !in_table)
    launch_moe_grouped_mma_f32(d_slot_act_, stride, d_segs_ + E, 1, max_rows, 0, d_sh_views_, 2, d_slot_down_, H, H,
                               w_.shared_inter, stream);
  if (!accumulate) return;
  const int shared_row0 = with_shared ? tk : -1;
  if (out_f32)
    launch_moe_accum_ordered_f32(out_f32, d_slot_down_, H, d_slot_row_, ids, weights, shared_row0, tokens, K, H, stream);
  else
    launch_moe_accum_ordered(out_bf16, d_slot_down_, H, d_slot_row_, ids, weights, shared_row0, tokens, K, H, stream);
}

// The prefill in phases (reference: route_prefill_rows / enqueue_prefill_phased / accumulate_prefill_rows,
// src/models/glm/moe_layer.cpp:843-904, for a caller that overlaps other work with the per-row ends of the layer): the
// router over a block of rows ahead of the chain, the chain over all rows without its accumulation, the accumulation
// per block of rows. The same kernels per row as enqueue_prefill: bitwise its output.
void GlmMoeLayer::route_prefill_rows(const uint16_t* x, size_t x_stride, int r0, int rows, hipStream_t stream) {
  if (rows <= 0) return;
  if (r0 < 0 || r0 > max_tokens_ - rows) throw std::invalid_argument("GlmMoeLayer: the row block exceeds the layer's max_tokens");
  if (!w_.router_gate) throw std::invalid_argument("GlmMoeLayer: the router gate is not bound");
  const size_t E = static_cast<size_t>(cfg_.n_experts), K = static_cast<size_t>(cfg_.top_k), at = static_cast<size_t>(r0);
  launch_moe_router_dots(x + at * x_stride, w_.router_gate, w_.router_bias, d_scores_ + at * E, d_biased_ + at * E, cfg_, rows,
                         stream);
  launch_moe_router_select(d_scores_ + at * E, d_biased_ + at * E, d_ids_ + at * K, d_weights_ + at * K, cfg_, rows, stream);
}
void GlmMoeLayer::enqueue_prefill_phased(const uint16_t* x, size_t x_stride, int tokens, hipStream_t stream) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  if (dense_shared()) throw std::invalid_argument("GlmMoeLayer: the phased prefill takes the shared expert as a segment");
  prefill_chain(x, x_stride, d_ids_, d_weights_, nullptr, nullptr, tokens, stream, has_shared(), /*accumulate=*/false);
}
void GlmMoeLayer::accumulate_prefill_rows(uint16_t* out_bf16, float* out_f32, int tokens, int r0, int rows, hipStream_t stream) {
  if (rows <= 0) return;
  check_tokens(tokens);
  if (out_bf16 == nullptr && out_f32 == nullptr) throw std::invalid_argument("GlmMoeLayer: no output buffer");
  if (r0 < 0 || r0 > tokens - rows) throw std::invalid_argument("GlmMoeLayer: the row block lies outside the batch");
  if (dense_shared()) throw std::invalid_argument("GlmMoeLayer: the phased prefill takes the shared expert as a segment");
  const int K = cfg_.top_k, H = cfg_.hidden;
  const size_t at = static_cast<size_t>(r0);
  const int shared_row0 = has_shared() ? tokens * K + r0 : -1;
  if (out_f32)
    launch_moe_accum_ordered_f32(out_f32 + at * H, d_slot_down_, H, d_slot_row_ + at * K, d_ids_ + at * K, d_weights_ + at * K,
                                 shared_row0, rows, K, H, stream);
  else
    launch_moe_accum_ordered(out_bf16 + at * H, d_slot_down_, H, d_slot_row_ + at * K, d_ids_ + at * K, d_weights_ + at * K,
                             shared_row0, rows, K, H, stream);
}

// The reference's W4A4 prefill chain (src/models/glm/moe_layer.cpp:1122-1135 the token rows' quantizer, :1217-1219
// gate / up over the routed row list, :1306-1316 SwiGLU inside the second quantizer when no shared segment rides
// along, :1268-1272 the down projection in bf16 or f32, :690 the accumulation from bf16 down rows).
void GlmMoeLayer::enqueue_prefill_routed_w4a4(const uint16_t* x, size_t x_stride, const int32_t* ids, const float* weights,
                                              uint16_t* out_bf16, float* out_f32, int tokens, hipStream_t stream,
                                              const float* act_scales_dev, bool f32_down) {
  if (tokens <= 0) return;
  check_tokens(tokens);
  if (out_bf16 == nullptr && out_f32 == nullptr) throw std::invalid_argument("GlmMoeLayer: no output buffer");
  if (w_.format != GlmExpertFormat::Nvfp4)
    throw std::invalid_argument("GlmMoeLayer: the activation-quantized path takes NVFP4 experts");
  const int K = cfg_.top_k, H = cfg_.hidden, I = cfg_.inter, E = cfg_.n_experts;
  if (H % 64 != 0 || I % 64 != 0)
    throw std::invalid_argument("GlmMoeLayer: the activation-quantized path needs hidden and inter in multiples of 64");
  const int tk = tokens * K;
  const bool dense = dense_shared();
  const bool seg_shared = has_shared() && !dense;   // the shared expert's rows keep BF16 activations behind the routed rows
  float* acc = dense ? (out_f32 ? out_f32 : d_acc_) : out_f32;
  uint16_t* rounded = dense ? nullptr : out_bf16;
  StreamFork fork{stream, side_, fork_, join_};
  if (dense) {
    fork.begin();
    dense_shared_chain(x, x_stride, tokens, side_);
  }
  launch_moe_segment(ids, tokens, K, E, d_rows_, d_slot_row_, d_segs_, stream);
  launch_quantize_rows_nvfp4(x, x_stride, tokens, H, d_q_codes_, d_q_scales_, d_q_gs_, stream, 0.f, act_scales_dev);
  launch_moe_grouped_w4a4_bf16(d_q_codes_, d_q_scales_, d_q_gs_, d_rows_, d_segs_, E, tokens, d_views_, 0, d_gate_, I, I, H,
                               stream);
  launch_moe_grouped_w4a4_bf16(d_q_codes_, d_q_scales_, d_q_gs_, d_rows_, d_segs_, E, tokens, d_views_, 1, d_up_, I, I, H,
                               stream);
  launch_swiglu_quantize_rows_nvfp4(d_gate_, d_up_, I, tk, I, cfg_.swiglu_limit, d_q_codes_, d_q_scales_, d_q_gs_, stream, 0.f,
                                    act_scales_dev ? act_scales_dev + 1 : nullptr);
  if (seg_shared) {
    const MoeExpertView* table = w_.shared_in_table ? d_views_ : d_sh_views_;
    const int SI = w_.shared_inter;
    const size_t stride = static_cast<size_t>(max_inter_);
    if (w_.shared_in_table)
      launch_moe_grouped_mma_gate_up_swiglu_fp4(x, x_stride, d_segs_ + E, 1, tokens, 0, table, d_slot_act_, stride, SI, H,
                                                cfg_.swiglu_limit, stream, d_rows_, fp4_group_);
    else
      launch_moe_grouped_mma_gate_up_swiglu(x, x_stride, d_segs_ + E, 1, tokens, 0, table, d_slot_act_, stride, SI, H,
                                            cfg_.swiglu_limit, stream, d_rows_);
    if (w_.shared_in_table)
      launch_moe_grouped_mma_fp4_f32(d_slot_act_, stride, d_segs_ + E, 1, tokens, 0, table, 2, d_slot_down_, H, H, SI, stream,
                                     nullptr, fp4_group_);
    else
      launch_moe_grouped_mma_f32(d_slot_act_, stride, d_segs_ + E, 1, tokens, 0, table, 2, d_slot_down_, H, H, SI, stream);
  }
  if (f32_down || seg_shared) {   // the shared rows are fp32: so are the routed ones (src/models/glm/moe_layer.cpp:1121)
    launch_moe_grouped_w4a4_f32(d_q_codes_, d_q_scales_, d_q_gs_, nullptr, d_segs_, E, tokens, d_views_, 2, d_slot_down_, H, H,
                                I, stream);
    const int shared_row0 = seg_shared ? tk : -1;
    if (acc)
      launch_moe_accum_ordered_f32(acc, d_slot_down_, H, d_slot_row_, ids, weights, shared_row0, tokens, K, H, stream);
    else
      launch_moe_accum_ordered(rounded, d_slot_down_, H, d_slot_row_, ids, weights, shared_row0, tokens, K, H, stream);
  } else {
    uint16_t* down = reinterpret_cast<uint16_t*>(d_slot_down_);
    launch_moe_grouped_w4a4_bf16(d_q_codes_, d_q_scales_, d_q_gs_, nullptr, d_segs_, E, tokens, d_views_, 2, down, H, H, I,
                                 stream);
    if (acc)
      launch_moe_accum_ordered_f32_bf16down(acc, down, H, d_slot_row_, ids, weights, tokens, K, H, stream);
    else
      launch_moe_accum_ordered_bf16down(rounded, down, H, d_slot_row_, ids, weights, tokens, K, H, stream);
  }
  if (dense) {
    fork.end();
    launch_moe_accum(acc, d_sh_down_, d_rows_id_, d_ones_, tokens, H, stream);
    if (!out_f32) launch_moe_round_bf16(out_bf16, acc, static_cast<int64_t>(tokens) * H, stream);
  }
}

}  // namespace dgpp

// ---- C wrappers -------------------------------------------------------------------------------------------
namespace {
thread_local std::string g_layer_error;
template <class Fn>
int guarded(Fn fn) {
  try {
    fn();
    return DGPP_OK;
  } catch (const std::invalid_argument& e) {
    g_layer_error = e.what();
    return DGPP_INVALID_ARGUMENT;
  } catch (const std::exception& e) {
    g_layer_error = e.what();
    return DGPP_RUNTIME_ERROR;
  }
}
dgpp::GlmMoeConfig cpp_config(const DgppMoeConfig& c) {
  dgpp::GlmMoeConfig g;
  g.hidden = c.hidden;
  g.inter = c.inter;
  g.n_experts = c.n_experts;
  g.top_k = c.top_k;
  g.n_shared_experts = c.n_shared_experts;
  g.routed_scaling_factor = c.routed_scaling_factor;
  g.norm_topk_prob = c.norm_topk_prob != 0;
  g.swiglu_limit = c.swiglu_limit;
  g.router_mode = static_cast<dgpp::MoeRouterMode>(c.router_mode);
  return g;
}
}  // namespace

struct DgppMoeLayer {
  dgpp::GlmMoeLayer impl;
  DgppMoeLayer(const dgpp::GlmMoeConfig& c, const dgpp::GlmMoeLayerWeights& w, int m) : impl(c, w, m) {}
};

extern "C" {

const char* dgpp_moe_layer_last_error(void) { return g_layer_error.c_str(); }

size_t dgpp_moe_layer_scratch_bytes(const DgppMoeConfig* cfg, int max_tokens, int shared_inter) {
  return dgpp::GlmMoeLayer::scratch_bytes(cpp_config(*cfg), max_tokens, shared_inter);
}

size_t dgpp_moe_layer_scratch_bytes_dense_shared(const DgppMoeConfig* cfg, int max_tokens, int shared_inter) {
  return dgpp::GlmMoeLayer::scratch_bytes(cpp_config(*cfg), max_tokens, shared_inter, true);
}

int dgpp_moe_layer_create(const DgppMoeLayerDesc* d, DgppMoeLayer** out) {
  return guarded([&] {
    if (!d || !out || !d->views) throw std::invalid_argument("moe_layer_create: null pointer");
    dgpp::GlmMoeLayerWeights w;
    w.format = static_cast<dgpp::GlmExpertFormat>(d->expert_format);
    const size_t n = (static_cast<size_t>(d->cfg.n_experts) + (d->shared_in_table ? 1 : 0)) * 3;
    w.views.assign(d->views, d->views + n);
    w.shared_in_table = d->shared_in_table != 0;
    w.shared_inter = d->shared_inter;
    for (int i = 0; i < 3; ++i) {
      w.sh_payload[i] = d->sh_payload[i];
      w.sh_scales[i] = d->sh_scales[i];
    }
    w.sh_rs = d->sh_rs;
    w.sh_cs = d->sh_cs;
    for (int i = 0; i < 3; ++i) w.sh_scales_e8m0[i] = d->sh_scales_e8m0[i];
    w.router_gate = d->router_gate;
    w.router_bias = d->router_bias;
    *out = new DgppMoeLayer(cpp_config(d->cfg), w, d->max_tokens);
  });
}

void dgpp_moe_layer_destroy(DgppMoeLayer* layer) { delete layer; }

int dgpp_moe_layer_enqueue_decode(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, uint16_t* out_bf16,
                                  float* out_f32, int tokens, void* stream) {
  return guarded([&] { l->impl.enqueue_decode(x, x_stride, out_bf16, out_f32, tokens, static_cast<hipStream_t>(stream)); });
}
int dgpp_moe_layer_enqueue_decode_scores(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, const float* scores,
                                         const float* biased, uint16_t* out_bf16, float* out_f32, int tokens,
                                         void* stream) {
  return guarded([&] {
    l->impl.enqueue_decode_scores(x, x_stride, scores, biased, out_bf16, out_f32, tokens, static_cast<hipStream_t>(stream));
  });
}
int dgpp_moe_layer_enqueue_decode_routed(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, const int32_t* ids,
                                         const float* weights, uint16_t* out_bf16, float* out_f32, int tokens,
                                         void* stream) {
  return guarded([&] {
    l->impl.enqueue_decode_routed(x, x_stride, ids, weights, out_bf16, out_f32, tokens, static_cast<hipStream_t>(stream));
  });
}
int dgpp_moe_layer_enqueue_grouped_routed(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, const int32_t* ids,
                                          const float* weights, uint16_t* out_bf16, float* out_f32, int tokens,
                                          void* stream) {
  return guarded([&] {
    l->impl.enqueue_grouped_routed(x, x_stride, ids, weights, out_bf16, out_f32, tokens, static_cast<hipStream_t>(stream));
  });
}
int dgpp_moe_layer_enqueue_prefill_routed(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, const int32_t* ids,
                                          const float* weights, uint16_t* out_bf16, float* out_f32, int tokens,
                                          void* stream) {
  return guarded([&] {
    l->impl.enqueue_prefill_routed(x, x_stride, ids, weights, out_bf16, out_f32, tokens, static_cast<hipStream_t>(stream));
  });
}
int dgpp_moe_layer_enqueue_prefill(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, uint16_t* out_bf16, float* out_f32,
                                   int tokens, void* stream) {
  return guarded([&] { l->impl.enqueue_prefill(x, x_stride, out_bf16, out_f32, tokens, static_cast<hipStream_t>(stream)); });
}
int dgpp_moe_layer_route_prefill_rows(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, int r0, int rows, void* stream) {
  return guarded([&] { l->impl.route_prefill_rows(x, x_stride, r0, rows, static_cast<hipStream_t>(stream)); });
}
int dgpp_moe_layer_enqueue_prefill_phased(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, int tokens, void* stream) {
  return guarded([&] { l->impl.enqueue_prefill_phased(x, x_stride, tokens, static_cast<hipStream_t>(stream)); });
}
int dgpp_moe_layer_accumulate_prefill_rows(DgppMoeLayer* l, uint16_t* out_bf16, float* out_f32, int tokens, int r0, int rows,
                                           void* stream) {
  return guarded([&] { l->impl.accumulate_prefill_rows(out_bf16, out_f32, tokens, r0, rows, static_cast<hipStream_t>(stream)); });
}
int dgpp_moe_layer_enqueue_prefill_routed_w4a4(DgppMoeLayer* l, const uint16_t* x, size_t x_stride, const int32_t* ids,
                                               const float* weights, uint16_t* out_bf16, float* out_f32, int tokens,
                                               void* stream, const float* act_scales_dev, int f32_down) {
  return guarded([&] {
    l->impl.enqueue_prefill_routed_w4a4(x, x_stride, ids, weights, out_bf16, out_f32, tokens,
                                        static_cast<hipStream_t>(stream), act_scales_dev, f32_down != 0);
  });
}
int dgpp_moe_layer_check(DgppMoeLayer* l, void* stream) {
  return guarded([&] { l->impl.check(static_cast<hipStream_t>(stream)); });
}
const DgppMoeExpertView* dgpp_moe_layer_views(const DgppMoeLayer* l) { return l->impl.views(); }
const int32_t* dgpp_moe_layer_ids(const DgppMoeLayer* l) { return l->impl.ids(); }
const float* dgpp_moe_layer_weights(const DgppMoeLayer* l) { return l->impl.weights(); }

}  // extern "C"
