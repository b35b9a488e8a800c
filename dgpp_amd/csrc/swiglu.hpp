// The SwiGLU epilogue shared by the fused gate/up kernels and the elementwise launcher.
// Rounding points follow the reference (src/kernels/glm_moe.cu:659-666): both dots rounded to bf16,
// the gate clamped above only, the up value on both sides, bf16(g * sigmoid(g)), bf16(t * u).
#pragma once

#include <hip/hip_runtime.h>

#include "numerics.hpp"

namespace dgpp_amd {

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ uint16_t swiglu_bf16(float gate_dot, float up_dot, float limit) {
  float g = bf16_to_f32(f32_to_bf16(gate_dot));
  float u = bf16_to_f32(f32_to_bf16(up_dot));
  if (g > limit) g = limit;
  u = fminf(fmaxf(u, -limit), limit);
  const uint16_t t = f32_to_bf16(g * sigmoid_f32(g));
  return f32_to_bf16(bf16_to_f32(t) * u);
}

// Eight bf16 gate / up pairs at once (one 16-byte vector each).
__device__ __forceinline__ uint4 swiglu_bf16x8(const uint4& gate, const uint4& up, float limit) {
  const uint32_t g[4] = {gate.x, gate.y, gate.z, gate.w}, u[4] = {up.x, up.y, up.z, up.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint16_t lo = swiglu_bf16(bits_f32(g[i] << 16), bits_f32(u[i] << 16), limit);
    const uint16_t hi = swiglu_bf16(bits_f32(g[i] & 0xFFFF0000u), bits_f32(u[i] & 0xFFFF0000u), limit);
    o[i] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

}  // namespace dgpp_amd
