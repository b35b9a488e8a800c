// Top-k expert selection of one token by one wavefront, whole score row in registers. Shared by the
// router's selection kernels and by the decode gate/up kernel that repeats the selection in every block.
// Reference counterpart: src/kernels/glm_moe.cu:314-329 (moe_router_select_kernel).
#pragma once

#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"
#include "numerics.hpp"

namespace dgpp_amd {
namespace rsel {

constexpr int kWaveSize = 64;

// The same selection for up to 64 * PER_LANE experts with the whole row in registers (expert e
// lives in lane e % 64, slot e / 64): no LDS, no barriers, DPP reductions inside 16-lane rows and
// four lane reads across them. A value's ordering key is a monotone unsigned image of the float
// (-0 folded into +0 first: they compare equal as floats; NaN maps to 0 and never wins); among
// equal keys the LOWEST id is taken — the strict '>' scan's outcome.
template <int kCtrl>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), kCtrl, 0xF, 0xF, true));
}
template <int kCtrl>
__device__ __forceinline__ float dpp_f32(float v) {
  return bits_f32(dpp_u32<kCtrl>(f32_bits(v)));
}
__device__ __forceinline__ float row_lane(float v, int lane) {
  return bits_f32(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(f32_bits(v)), lane)));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  return (row_lane(v, 0) + row_lane(v, 16)) + (row_lane(v, 32) + row_lane(v, 48));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, dpp_f32<0xB1>(v));
  v = fmaxf(v, dpp_f32<0x4E>(v));
  v = fmaxf(v, dpp_f32<0x141>(v));
  v = fmaxf(v, dpp_f32<0x140>(v));
  return fmaxf(fmaxf(row_lane(v, 0), row_lane(v, 16)), fmaxf(row_lane(v, 32), row_lane(v, 48)));
}
__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t lane_u32(uint32_t v, int lane) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane));
}
// Wave-wide max / min of one value per lane, the same in every lane on return: a butterfly inside each row of
// 16 lanes, then row 0 -> 1 and 2 -> 3, then row 1 -> 2, 3 (row broadcasts), and lane 63 read back.
template <bool kMax>
__device__ __forceinline__ uint32_t wave_reduce_u32(uint32_t v) {
  auto op = [](uint32_t a, uint32_t b) { return kMax ? (a > b ? a : b) : (a < b ? a : b); };
  v = op(v, dpp_u32<0xB1>(v));
  v = op(v, dpp_u32<0x4E>(v));
  v = op(v, dpp_u32<0x141>(v));
  v = op(v, dpp_u32<0x140>(v));
  const int i = static_cast<int>(v);
  v = op(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(i, i, 0x142, 0xA, 0xF, false)));   // row_bcast:15 into rows 1, 3
  const int k = static_cast<int>(v);
  v = op(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(k, k, 0x143, 0xC, 0xF, false)));   // row_bcast:31 into rows 2, 3
  return lane_u32(v, 63);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) { return wave_reduce_u32<true>(v); }
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) { return wave_reduce_u32<false>(v); }
__device__ __forceinline__ uint32_t order_key(float v) {
  if (v != v) return 0u;                       // NaN: below every real key
  const uint32_t u = f32_bits(v + 0.0f);       // -0 -> +0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One wavefront selects for one token. On return lane p < top_k holds the token's p-th expert in
// ascending id order and its final weight; no private arrays, no LDS.
// kAddBias: `biased` holds the per-expert bias and the ranking value is scores[e] + bias[e], formed here; the weights
// are then score / max(sum, 1e-20) * scaling, never narrowed (the MiniMax router, src/kernels/minimax.cu:409-440).
template <int kMode, int PER_LANE, bool kAddBias = false>
__device__ __forceinline__ void select_token(const float* __restrict__ scores, const float* __restrict__ biased,
                                             int n_experts, int top_k, float scaling, int norm_topk, int lane,
                                             int& out_id, float& out_w) {
  float sc[PER_LANE];
  uint32_t key[PER_LANE];
  {
    // every load is issued before the first is waited for (dead slots re-read the last expert): one trip to memory
    float raw_s[PER_LANE], raw_b[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      const int e = min(lane + j * kWaveSize, n_experts - 1);
      raw_s[j] = scores[e];
      raw_b[j] = biased[e];
    }
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      const bool live = lane + j * kWaveSize < n_experts;
      sc[j] = live ? raw_s[j] : -INFINITY;
      key[j] = live ? order_key(kAddBias ? raw_s[j] + raw_b[j] : raw_b[j]) : 0u;
    }
  }
  if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) {
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) m = fmaxf(m, sc[j]);
    m = wave_max_dpp(m);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      sc[j] = lane + j * kWaveSize < n_experts ? expf(sc[j] - m) : 0.f;
      sum += sc[j];
    }
    sum = wave_sum_dpp(sum);
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) sc[j] = sc[j] / sum;
  }
  // Pick r lands in lane r. A round is two wave-wide reductions on the vector side: the maximum key, then the
  // LOWEST expert id among the lanes and slots that hold it (ids are slot-major, e = lane + 64 * slot).
  int my_id = INT_MAX;
  float my_w = 0.f;
  for (int r = 0; r < top_k; ++r) {
    uint32_t m = key[0];
#pragma unroll
    for (int j = 1; j < PER_LANE; ++j) m = m > key[j] ? m : key[j];
    const uint32_t top = wave_max_u32(m);
    uint32_t cand = 0xFFFFFFFFu;
#pragma unroll
    for (int j = PER_LANE - 1; j >= 0; --j) cand = key[j] == top ? static_cast<uint32_t>(lane + j * kWaveSize) : cand;
    int best = static_cast<int>(wave_min_u32(cand));
    if (top == 0u || best >= n_experts) best = 0;   // a row of NaN keys: stay in bounds
    float mine = 0.f;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      const bool hit = lane + j * kWaveSize == best;
      mine = hit ? sc[j] : mine;
      key[j] = hit ? 0u : key[j];                   // taken: below every real key
    }
    const float w = row_lane(mine, best & (kWaveSize - 1));
    if (lane == r) {
      my_id = best;
      my_w = w;
    }
  }
  // Ascending expert id, stable in pick order: rank of lane's pick, then the inverse permutation.
  int rank = 0;
  for (int i = 0; i < top_k; ++i) {
    const int oid = __builtin_amdgcn_readlane(my_id, i);
    rank += (oid < my_id) || (oid == my_id && i < lane);
  }
  int src = 0;
  for (int i = 0; i < top_k; ++i)
    if (__builtin_amdgcn_readlane(rank, i) == lane) src = i;
  const int sid = __shfl(my_id, src);
  const float sw = __shfl(my_w, src);
  float denom = 0.f;
  for (int i = 0; i < top_k; ++i) denom += row_lane(sw, i);   // fp32 adds in id order
  if (kAddBias) denom = fmaxf(denom, 1e-20f);
  else denom += 1e-20f;
  float w = norm_topk ? (sw / denom) * scaling : sw * scaling;
  if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) w = bf16_to_f32(f32_to_bf16(w));
  out_id = sid;
  out_w = w;
}

}  // namespace rsel
}  // namespace dgpp_amd
