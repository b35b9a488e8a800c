// A compiled host program over include/dgpp_amd.hpp: reference-style C++ calling the dgpp::launch_* names on a real
// GPU, apart from the stream type unchanged. Built by dgpp_amd/build.py (dgpp_amd/lib/dgpp_host_program), run by
// tests/test_gpu_host_program.py as a subprocess; exit status 0 = every check held, 2 = no device.
//
// (i)  the reference's geometry-rejection tests of the dense FP4 GEMV, ported one to one
//      (tests/cuda/fp4_gemv_test.cu:276-313 MXFP4 set, :398-415 NVFP4 set): std::invalid_argument before any launch;
// (ii) the reference's decode call order (src/models/glm/moe_layer.cpp:1641-1677: router, slot order, fused gate/up +
//      SwiGLU, down, accumulation) stitched from the shim's launchers, bit for bit the layer driver's
//      dgpp_moe_layer_enqueue_decode on the same weights and rows.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/dgpp_amd.hpp"
#include "../../include/dgpp_amd_layer.h"

namespace {

int g_failed = 0;
void require(bool ok, const char* what) {
  if (ok) return;
  std::printf("[FAIL] %s\n", what);
  ++g_failed;
}
void hip_ok(hipError_t e, const char* what) {
  if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// A device copy of a host vector (freed with the program).
template <class T>
T* upload(const std::vector<T>& v) {
  T* d = nullptr;
  hip_ok(hipMalloc(&d, v.size() * sizeof(T) + 16), "hipMalloc");
  hip_ok(hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice), "upload");
  return d;
}
template <class T>
T* device_zeros(size_t n) {
  T* d = nullptr;
  hip_ok(hipMalloc(&d, n * sizeof(T) + 16), "hipMalloc");
  hip_ok(hipMemset(d, 0, n * sizeof(T)), "hipMemset");
  return d;
}
template <class T>
std::vector<T> download(const T* d, size_t n) {
  std::vector<T> v(n);
  hip_ok(hipMemcpy(v.data(), d, n * sizeof(T), hipMemcpyDeviceToHost), "download");
  return v;
}

// One FP4 matrix on the device: MXFP4 (group 32, no global) or NVFP4 (group 16, device global = 1 / weight_scale_2).
struct DevFp4 {
  dgpp::GlmFp4Matrix view{};
};
DevFp4 make_fp4(uint64_t seed, int n, int k, int group) {
  std::vector<float> w(static_cast<size_t>(n) * k);
  dgpp_fill_normal_f32(seed, 0.f, 0.05f, static_cast<int64_t>(w.size()), w.data(), 1);
  std::vector<uint8_t> payload(static_cast<size_t>(n) * k / 2), scales(static_cast<size_t>(n) * k / group);
  DevFp4 m;
  if (group == 32) {
    dgpp_encode_mxfp4(w.data(), n, k, payload.data(), scales.data(), 1);
  } else {
    const float ws2 = dgpp_encode_nvfp4(w.data(), n, k, payload.data(), scales.data(), 1);
    m.view.global_scale = upload(std::vector<float>{1.0f / ws2});
  }
  m.view.payload = upload(payload);
  m.view.scales = upload(scales);
  m.view.rows = n;
  m.view.cols = k;
  m.view.scale_group = group;
  return m;
}

// ---- (i) geometry rejection --------------------------------------------------------------------------------------
bool rejects(int k, int group) {
  const int n = 8;
  DevFp4 w = make_fp4(0x3BAD + static_cast<uint64_t>(k), n, k, group);
  std::vector<uint16_t> act(static_cast<size_t>(k));
  dgpp_fill_normal_bf16(7, 0.f, 1.f, k, act.data(), 1);
  uint16_t* d_act = upload(act);
  uint16_t* d_out = device_zeros<uint16_t>(n);
  try {
    dgpp::launch_fp4_gemv_bf16(d_act, static_cast<size_t>(k), w.view, d_out, 1, n, k, nullptr);
    hip_ok(hipDeviceSynchronize(), "sync");
  } catch (const std::invalid_argument&) {
    return true;
  }
  return false;
}
void geometry_contract() {
  // tests/cuda/fp4_gemv_test.cu:276-313
  require(rejects(48, 32), "mxfp4 k=48 rejected (not a multiple of 32)");
  require(rejects(3072, 32), "mxfp4 k=3072 rejected (not in the MXFP4 compiled set)");
  require(!rejects(576, 32), "mxfp4 k=576 accepted (world-4 down)");
  require(!rejects(1152, 32), "mxfp4 k=1152 accepted (world-2 down)");
  require(!rejects(2304, 32), "mxfp4 k=2304 accepted (world-1 down)");
  require(!rejects(4096, 32), "mxfp4 k=4096 accepted (the MiMo gate/up)");
  require(!rejects(2048, 32), "mxfp4 k=2048 accepted (the MiMo world-1 down)");
  {
    DevFp4 w = make_fp4(0x3BAE, 8, 1024, 16);
    dgpp::GlmFp4Matrix v = w.view;
    v.global_scale = nullptr;
    uint16_t* act = device_zeros<uint16_t>(1024);
    uint16_t* out = device_zeros<uint16_t>(8);
    bool refused = false;
    try {
      dgpp::launch_fp4_gemv_bf16(act, 1024, v, out, 1, 8, 1024, nullptr);
    } catch (const std::invalid_argument&) {
      refused = true;
    }
    require(refused, "an NVFP4 view without a global scale is refused");
  }
  // tests/cuda/fp4_gemv_test.cu:398-415
  require(rejects(48, 16), "nvfp4 k=48 rejected (not a multiple of 32)");
  require(rejects(96, 16), "nvfp4 k=96 rejected (not in the compiled set)");
  require(!rejects(1536, 16), "nvfp4 k=1536 accepted");
  require(rejects(8192, 16), "nvfp4 k=8192 rejected (not in the compiled set)");
  require(!rejects(2048, 16), "nvfp4 k=2048 accepted");
  require(!rejects(5120, 16), "nvfp4 k=5120 accepted");
  std::printf("[ OK ] fp4 gemv geometry contract enforced through dgpp::launch_fp4_gemv_bf16\n");
}

// ---- (ii) the decode call order ------------------------------------------------------------------------------------
void decode_call_order(int group, int tokens) {
  dgpp::GlmMoeConfig cfg;
  cfg.hidden = 1024;
  cfg.inter = 256;
  cfg.n_experts = 32;
  cfg.top_k = 8;
  cfg.n_shared_experts = 0;
  cfg.routed_scaling_factor = 1.0f;
  cfg.swiglu_limit = INFINITY;
  cfg.router_mode = dgpp::MoeRouterMode::SoftmaxTopk;
  const int H = cfg.hidden, I = cfg.inter, E = cfg.n_experts, K = cfg.top_k, T = tokens;
  std::vector<dgpp::MoeExpertView> views;
  for (int e = 0; e < E; ++e) {
    views.push_back(dgpp::expert_view_of(make_fp4(1000 + 3 * e, I, H, group).view));
    views.push_back(dgpp::expert_view_of(make_fp4(1001 + 3 * e, I, H, group).view));
    views.push_back(dgpp::expert_view_of(make_fp4(1002 + 3 * e, H, I, group).view));
  }
  std::vector<uint16_t> x(static_cast<size_t>(T) * H), gate(static_cast<size_t>(E) * H);
  dgpp_fill_normal_bf16(11 + T, 0.f, 1.f, static_cast<int64_t>(x.size()), x.data(), 1);
  dgpp_fill_normal_bf16(12, 0.f, 0.05f, static_cast<int64_t>(gate.size()), gate.data(), 1);
  const uint16_t* d_x = upload(x);
  const uint16_t* d_gate = upload(gate);

  // the layer driver
  DgppMoeLayerDesc desc{};
  desc.cfg = cfg.c_config();
  desc.expert_format = group == 32 ? DGPP_EXPERTS_MXFP4 : DGPP_EXPERTS_NVFP4;
  desc.max_tokens = T;
  desc.views = views.data();
  desc.router_gate = d_gate;
  DgppMoeLayer* layer = nullptr;
  if (dgpp_moe_layer_create(&desc, &layer) != DGPP_OK) throw std::runtime_error(dgpp_moe_layer_last_error());
  uint16_t* d_want = device_zeros<uint16_t>(static_cast<size_t>(T) * H);
  if (dgpp_moe_layer_enqueue_decode(layer, d_x, static_cast<size_t>(H), d_want, nullptr, T, nullptr) != DGPP_OK)
    throw std::runtime_error(dgpp_moe_layer_last_error());
  hip_ok(hipDeviceSynchronize(), "sync");

  // the same step as the reference's model code writes it (src/models/glm/moe_layer.cpp:1476, 1555-1560, 1641-1677)
  hipStream_t stream = nullptr;
  hip_ok(hipStreamCreate(&stream), "stream");
  const int slots = T * (K + 1);
  const dgpp::MoeExpertView* d_views = upload(views);
  int32_t* d_ids = device_zeros<int32_t>(static_cast<size_t>(T) * K);
  float* d_weights = device_zeros<float>(static_cast<size_t>(T) * K);
  float* d_scores = device_zeros<float>(static_cast<size_t>(T) * E);
  float* d_biased = device_zeros<float>(static_cast<size_t>(T) * E);
  int32_t* d_order = device_zeros<int32_t>(static_cast<size_t>(slots));
  uint16_t* d_act = device_zeros<uint16_t>(static_cast<size_t>(slots) * I);
  float* d_down = device_zeros<float>(static_cast<size_t>(slots) * H);
  float* d_acc = device_zeros<float>(static_cast<size_t>(T) * H);
  uint16_t* d_out = device_zeros<uint16_t>(static_cast<size_t>(T) * H);
  int* d_counter = device_zeros<int>(2);
  dgpp::launch_moe_router(d_x, d_gate, nullptr, d_ids, d_weights, d_scores, d_biased, cfg, T, stream);
  const int32_t* order = nullptr;
  if (T > 1) {
    dgpp::launch_moe_slot_order(d_ids, d_order, slots, K, E, stream);
    order = d_order;
  }
  dgpp::launch_moe_slot_gate_up_swiglu_fp4(d_x, static_cast<size_t>(H), d_ids, order, d_views, I, H, 0, 0, nullptr, nullptr,
                                           nullptr, nullptr, d_act, I, slots, K, cfg.swiglu_limit, stream, -1, group);
  dgpp::launch_moe_slot_down_fp4(d_act, static_cast<size_t>(I), d_ids, order, d_views, H, I, 0, 0, nullptr, nullptr, d_down, H,
                                 slots, K, stream, -1, group, 7, 7, d_counter);
  dgpp::launch_moe_slot_accum_routed_f32(d_acc, d_down, d_weights, T, H, K, stream);
  dgpp::launch_moe_round_bf16(d_out, d_acc, static_cast<int64_t>(T) * H, stream);
  hip_ok(hipStreamSynchronize(stream), "sync");

  const auto want = download(d_want, static_cast<size_t>(T) * H), got = download(d_out, static_cast<size_t>(T) * H);
  require(std::memcmp(want.data(), got.data(), want.size() * 2) == 0, "stitched decode order == the layer driver, bit for bit");
  bool nonzero = false;
  for (uint16_t v : got) nonzero = nonzero || (v & 0x7FFFu) != 0;
  require(nonzero, "the layer's output is not all zeros");
  dgpp_moe_layer_destroy(layer);
  hip_ok(hipStreamDestroy(stream), "stream");
  std::printf("[ OK ] decode call order stitched from dgpp::launch_* (%s, %d token%s) is bitwise the layer driver\n",
              group == 32 ? "MXFP4" : "NVFP4", T, T == 1 ? "" : "s");
}

}  // namespace

int main() {
  int devices = 0;
  if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
    std::printf("[SKIP] no device\n");
    return 2;
  }
  try {
    geometry_contract();
    decode_call_order(32, 4);
    decode_call_order(32, 1);
    decode_call_order(16, 3);
  } catch (const std::exception& e) {
    std::printf("[FAIL] exception: %s\n", e.what());
    return 1;
  }
  if (g_failed) return 1;
  std::printf("host program: all checks passed\n");
  return 0;
}
