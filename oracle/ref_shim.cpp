// C entry points around the REFERENCE's own host oracle and codecs, compiled from the
// reference's sources where they lie (see the Makefile: nothing of the reference is copied
// into this repository; the output goes to oracle/_ref/ only).
//
// TEST INFRASTRUCTURE ONLY: used to validate oracle/dgpp_oracle.cpp and to write the small
// golden fixtures under tests/golden/. It exists only where the reference checkout exists.
#include <cstdint>
#include <cstring>
#include <exception>
#include <vector>

#include "common/dtypes.hpp"
#include "kernels/latent_format.hpp"
#include "loaders/fp8_quant.hpp"
#include "loaders/nvfp4_quant.hpp"
#include "models/glm/moe_reference.hpp"
#include "models/minimax/reference.hpp"

using namespace dgpp;

namespace {
GlmMoeConfig make_cfg(int hidden, int inter, int experts, int top_k, int mode, float scaling, int norm,
                      float limit) {
  GlmMoeConfig c;
  c.hidden = hidden;
  c.inter = inter;
  c.n_experts = experts;
  c.top_k = top_k;
  c.routed_scaling_factor = scaling;
  c.norm_topk_prob = norm != 0;
  c.swiglu_limit = limit;
  c.router_mode = mode == 1 ? MoeRouterMode::SoftmaxTopk
                            : (mode == 2 ? MoeRouterMode::SqrtSoftplusBias : MoeRouterMode::SigmoidBias);
  return c;
}
}  // namespace

extern "C" {

float ref_bf16_to_f32(uint16_t b) { return bf16_bits_to_float(b); }
uint16_t ref_f32_to_bf16(float f) { return float_to_bf16_bits(f); }
float ref_e4m3_to_f32(uint8_t v) { return fp8_e4m3_bits_to_float(v); }
uint8_t ref_f32_to_e4m3(float f) { return float_to_fp8_e4m3_bits(f); }
float ref_e2m1_to_f32(uint8_t v) { return fp4_e2m1_bits_to_float(v); }
uint8_t ref_f32_to_e2m1(float f) { return float_to_fp4_e2m1_bits(f); }
float ref_e8m0_to_f32(uint8_t v) { return e8m0_byte_to_float(v); }
uint8_t ref_e8m0_ceil_log2(float f) { return e8m0_ceil_log2_byte(f); }

float ref_nvfp4_tensor_scale(float amax) { return nvfp4_tensor_scale(amax); }
void ref_nvfp4_encode_row(const float* row, int64_t cols, float ws2, uint8_t* payload, uint8_t* scales) {
  nvfp4_encode_row(row, cols, ws2, payload, scales);
}
void ref_fp8_encode_block128(const uint16_t* src, int64_t rows, int64_t cols, uint8_t* payload, float* scales) {
  fp8_quant::encode_block128(src, static_cast<size_t>(cols), rows, cols, payload, scales, 1);
}

// The reference's MiniMax routing statement (src/models/minimax/reference.cpp:96-113) for one row of logits.
int ref_minimax_route(const float* logits, const float* bias, int experts, int topk, float factor, int32_t* ids,
                      float* weights) {
  try {
    std::vector<int> i;
    std::vector<float> w;
    dgpp::minimax_ref::route(logits, bias, experts, topk, factor, i, w);
    for (int j = 0; j < topk; ++j) {
      ids[j] = i[static_cast<size_t>(j)];
      weights[j] = w[static_cast<size_t>(j)];
    }
    return 0;
  } catch (const std::exception&) {
    return 1;
  }
}

// Router oracle: returns 0, or 1 when the reference threw.
int ref_router(const uint16_t* hidden, const uint16_t* gate, const float* bias, int mode, int tokens,
               int experts, int hidden_dim, int top_k, float scaling, int norm, int32_t* ids,
               float* weights, double* biased) {
  try {
    GlmMoeConfig c = make_cfg(hidden_dim, 64, experts, top_k, mode, scaling, norm, 10.f);
    GlmMoeRouterRef r;
    glm_moe_ref_router(hidden, gate, bias, c, tokens, r);
    std::memcpy(ids, r.ids.data(), r.ids.size() * sizeof(int32_t));
    std::memcpy(weights, r.weights.data(), r.weights.size() * sizeof(float));
    if (biased) std::memcpy(biased, r.biased.data(), r.biased.size() * sizeof(double));
    return 0;
  } catch (const std::exception&) {
    return 1;
  }
}

// Full layer oracle. fp8 vectors: the routed matrices (when fp4 == 0) then the shared triple
// (when shared_fp4 == 0); fp4 vectors: the routed matrices then the shared triple (shared_fp4).
int ref_moe_forward(const uint16_t* hidden, int tokens, int hidden_dim, int inter, int experts, int top_k,
                    int mode, float scaling, int norm, float limit, const uint16_t* router_gate,
                    const float* router_bias, const uint8_t* payloads, int64_t n_payloads,
                    const float* scales, int64_t n_scales, int fp4, int shared_fp4, int fp4_group,
                    const uint8_t* fp4_payloads, int64_t n_fp4_payloads, const uint8_t* fp4_scales,
                    int64_t n_fp4_scales, const float* fp4_globals, int64_t n_fp4_globals, uint16_t* out) {
  try {
    GlmMoeConfig c = make_cfg(hidden_dim, inter, experts, top_k, mode, scaling, norm, limit);
    GlmMoeHostWeights w;
    w.router_gate.assign(router_gate, router_gate + static_cast<size_t>(experts) * hidden_dim);
    if (router_bias) w.router_bias.assign(router_bias, router_bias + experts);
    else w.router_bias.assign(static_cast<size_t>(experts), 0.f);
    w.payloads.assign(payloads, payloads + n_payloads);
    w.scales.assign(scales, scales + n_scales);
    w.nvfp4 = fp4 != 0;
    w.shared_nvfp4 = shared_fp4 != 0;
    w.fp4_group = fp4_group;
    if (fp4) {
      w.fp4_payloads.assign(fp4_payloads, fp4_payloads + n_fp4_payloads);
      w.fp4_scales.assign(fp4_scales, fp4_scales + n_fp4_scales);
      if (fp4_globals) w.fp4_globals.assign(fp4_globals, fp4_globals + n_fp4_globals);
    }
    std::vector<uint16_t> o;
    glm_moe_ref_forward(hidden, w, c, tokens, o);
    std::memcpy(out, o.data(), o.size() * sizeof(uint16_t));
    return 0;
  } catch (const std::exception&) {
    return 1;
  }
}

// The same oracle with the layer's weights kept between calls (an FP4 layer: the routed matrices then the
// shared triple), so that a timed pass is the reference's forward alone and not the copy of its weights.
struct RefLayer {
  GlmMoeConfig cfg;
  GlmMoeHostWeights w;
};

void* ref_moe_layer_create(int hidden_dim, int inter, int experts, int top_k, int mode, float scaling, int norm,
                           float limit, const uint16_t* router_gate, const float* router_bias, int fp4_group,
                           const uint8_t* fp4_payloads, int64_t n_fp4_payloads, const uint8_t* fp4_scales,
                           int64_t n_fp4_scales, const float* fp4_globals, int64_t n_fp4_globals) {
  try {
    auto* l = new RefLayer();
    l->cfg = make_cfg(hidden_dim, inter, experts, top_k, mode, scaling, norm, limit);
    l->w.router_gate.assign(router_gate, router_gate + static_cast<size_t>(experts) * hidden_dim);
    if (router_bias) l->w.router_bias.assign(router_bias, router_bias + experts);
    else l->w.router_bias.assign(static_cast<size_t>(experts), 0.f);
    l->w.nvfp4 = true;
    l->w.shared_nvfp4 = true;
    l->w.fp4_group = fp4_group;
    l->w.fp4_payloads.assign(fp4_payloads, fp4_payloads + n_fp4_payloads);
    l->w.fp4_scales.assign(fp4_scales, fp4_scales + n_fp4_scales);
    if (fp4_globals) l->w.fp4_globals.assign(fp4_globals, fp4_globals + n_fp4_globals);
    return l;
  } catch (const std::exception&) {
    return nullptr;
  }
}

int ref_moe_layer_forward(const void* layer, const uint16_t* hidden, int tokens, uint16_t* out) {
  try {
    const auto* l = static_cast<const RefLayer*>(layer);
    std::vector<uint16_t> o;
    glm_moe_ref_forward(hidden, l->w, l->cfg, tokens, o);
    std::memcpy(out, o.data(), o.size() * sizeof(uint16_t));
    return 0;
  } catch (const std::exception&) {
    return 1;
  }
}

void ref_moe_layer_destroy(void* layer) { delete static_cast<RefLayer*>(layer); }

}  // extern "C"
