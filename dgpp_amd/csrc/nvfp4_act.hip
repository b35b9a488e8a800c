// The activation side of the W4A4 NVFP4 form: BF16 rows -> NVFP4 (e2m1 codes, one e4m3 scale per 16 elements, one
// fp32 global per row), alone or with the MoE's SwiGLU computed on the way, and the C entry points of the grouped
// W4A4 GEMM (its kernel is the matrix-core grouped kernel with NVFP4 activation rows: gemv_mfma_kernels.hpp).
//
// Reference: src/kernels/moe_w4a4.{hpp,cu} (quantize_rows_nvfp4_kernel :139-236, launchers :598-634, the grouped GEMM
// :239-442 and its launcher :636-715). The quantizer's recipe is a chain of single IEEE fp32 operations
//   global = static > 0 ? static : amax > 0 ? amax / (6 * 448) : 1
//   scale  = e4m3_rne_sat(amax16 / (6 * global));  q = 1 / (float(scale) * global);  code = e2m1_rne_sat(x * q)
// and is reproduced bit for bit. On this chip the GEMM multiplies the exactly decoded operands on the BF16 matrix core
// (the block-scaled FP4 instruction takes one power-of-two scale per 32 elements, NVFP4 carries an e4m3 per 16).
//
// Shape of the quantizer: one block per row; a lane owns whole 16-element groups (32 contiguous bytes of the row: two
// 16-byte loads) and keeps them as packed BF16 words between the row-maximum reduction and the encoding, so the row is
// read once. Groups are dealt to lanes round-robin: a wavefront's loads cover 2 KB of contiguous row per step.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include <string>

#include "../../include/dgpp_amd.h"
#include "capi_errors.hpp"
#include "gemv_kernels.hpp"
#include "numerics.hpp"
#include "swiglu.hpp"

namespace dgpp_amd {
namespace {

constexpr int kQuantThreads = 256;

__device__ __forceinline__ float qmax_dpp(float v) {   // maximum over the wavefront, in every lane
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// SwiGLU forms of the fused quantizer: the MoE's (two BF16 roundings, asymmetric clamp: swiglu.hpp) and the dense
// MLP's of the Qwen family (silu as g / (1 + exp(-g)), one rounding of the product, no clamp;
// src/kernels/moe_w4a4.cu:117-123).
__device__ __forceinline__ uint16_t swiglu_qwen_bits(uint16_t g_bits, uint16_t u_bits) {
  const float g = bf16_to_f32(g_bits), u = bf16_to_f32(u_bits);
  const float s = g / (1.0f + expf(-g));
  return f32_to_bf16(s * u);
}

struct QuantArgs {
  const uint16_t* x;        // rows (the gate rows of the fused form)
  const uint16_t* up;       // fused form only
  size_t stride;            // elements
  int rows, k;
  uint8_t* codes;           // [rows, k / 2]
  uint8_t* scales;          // [rows, scale_stride]
  size_t scale_stride;
  float* gs;                // [rows]
  float static_gs;
  const float* static_gs_dev;
  float limit;
  int aligned;              // rows may be read as 16-byte vectors
};

// MODE 0: plain rows; 1: the MoE's SwiGLU of (x, up); 2: the Qwen dense MLP's SwiGLU.
// RECIPE 0: the scale chain of src/kernels/moe_w4a4.cu (above). RECIPE 1: the per-token dynamic producer of
// src/kernels/minimax_native_moe.cu:36-85 (MODE 0 only), whose chain multiplies by reciprocals:
//   decode = amax * (1 / 2688);  encode = amax == 0 ? FLT_MAX : 1 / decode;  global = decode
//   scale  = e4m3_rne_sat(encode * (amax16 * (1 / 6)));  inv = float(scale) == 0 ? 0 : 1 / (float(scale) * (1 / encode))
//   code   = e2m1_rne_sat(x * inv)      (a zero scale leaves signed zeros: the sign bit of x survives in the code)
// Every reciprocal here is the correctly rounded one; the reference takes NVIDIA's approximate instruction, whose last
// bit is its own.
template <int GPT, int MODE, int RECIPE = 0>
__global__ __launch_bounds__(kQuantThreads) void nvfp4_quantize_rows_kernel(QuantArgs a) {
  __shared__ float wave_max[kQuantThreads / 64];
  const int row = static_cast<int>(blockIdx.x);
  const int groups = a.k / 16;
  const uint16_t* xr = a.x + static_cast<size_t>(row) * a.stride;
  const uint16_t* ur = MODE != 0 ? a.up + static_cast<size_t>(row) * a.stride : nullptr;
  uint32_t w[GPT][8];   // the lane's groups as packed BF16 pairs (after the SwiGLU in the fused forms)
  float gmax[GPT];
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < GPT; ++j) {
    const int g = static_cast<int>(threadIdx.x) + j * kQuantThreads;
    gmax[j] = 0.f;
    if (g < groups) {
      if (MODE != 0 || a.aligned) {
        const uint4* src = reinterpret_cast<const uint4*>(xr + g * 16);
        const uint4 v0 = src[0], v1 = src[1];
        w[j][0] = v0.x, w[j][1] = v0.y, w[j][2] = v0.z, w[j][3] = v0.w;
        w[j][4] = v1.x, w[j][5] = v1.y, w[j][6] = v1.z, w[j][7] = v1.w;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          w[j][i] = static_cast<uint32_t>(xr[g * 16 + 2 * i]) | (static_cast<uint32_t>(xr[g * 16 + 2 * i + 1]) << 16);
      }
      if constexpr (MODE != 0) {
        const uint4* us = reinterpret_cast<const uint4*>(ur + g * 16);
        const uint4 u0 = us[0], u1 = us[1];
        const uint32_t u[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint16_t gl = static_cast<uint16_t>(w[j][i] & 0xFFFFu), gh = static_cast<uint16_t>(w[j][i] >> 16);
          const uint16_t ul = static_cast<uint16_t>(u[i] & 0xFFFFu), uh = static_cast<uint16_t>(u[i] >> 16);
          uint16_t lo, hi;
          if constexpr (MODE == 1) {
            lo = swiglu_bf16(bf16_to_f32(gl), bf16_to_f32(ul), a.limit);
            hi = swiglu_bf16(bf16_to_f32(gh), bf16_to_f32(uh), a.limit);
          } else {
            lo = swiglu_qwen_bits(gl, ul);
            hi = swiglu_qwen_bits(gh, uh);
          }
          w[j][i] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
        gmax[j] = fmaxf(gmax[j], fmaxf(fabsf(bits_f32(w[j][i] << 16)), fabsf(bits_f32(w[j][i] & 0xFFFF0000u))));
      amax = fmaxf(amax, gmax[j]);
    }
  }
  amax = qmax_dpp(amax);
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  float row_amax = wave_max[0];
#pragma unroll
  for (int v = 1; v < kQuantThreads / 64; ++v) row_amax = fmaxf(row_amax, wave_max[v]);
  uint8_t* scale_row = a.scales + static_cast<size_t>(row) * a.scale_stride;
  uint8_t* code_row = a.codes + static_cast<size_t>(row) * (a.k / 2);
  if constexpr (RECIPE == 1) {
    const float decode = row_amax * (1.f / (6.f * 448.f));
    const float encode = row_amax == 0.f ? 3.402823466e+38f : 1.f / decode;
    if (threadIdx.x == 0) a.gs[row] = decode;
#pragma unroll
    for (int j = 0; j < GPT; ++j) {
      const int g = static_cast<int>(threadIdx.x) + j * kQuantThreads;
      if (g >= groups) continue;
      const uint8_t sb = f32_to_e4m3(encode * (gmax[j] * (1.f / 6.f)));
      const float sv = e4m3_to_f32(sb);
      const float inv = sv == 0.f ? 0.f : 1.f / (sv * (1.f / encode));
      uint32_t c[2] = {0u, 0u};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t lo = f32_to_e2m1(bits_f32(w[j][i] << 16) * inv);
        const uint32_t hi = f32_to_e2m1(bits_f32(w[j][i] & 0xFFFF0000u) * inv);
        c[i >> 2] |= (lo | (hi << 4)) << (8 * (i & 3));
      }
      scale_row[g] = sb;
      *reinterpret_cast<uint2*>(code_row + g * 8) = make_uint2(c[0], c[1]);
    }
    return;
  }
  const float sg = a.static_gs_dev != nullptr ? *a.static_gs_dev : a.static_gs;
  const float global = sg > 0.f ? sg : (row_amax > 0.f ? row_amax / (6.f * 448.f) : 1.f);
  if (threadIdx.x == 0) a.gs[row] = global;
#pragma unroll
  for (int j = 0; j < GPT; ++j) {
    const int g = static_cast<int>(threadIdx.x) + j * kQuantThreads;
    if (g >= groups) continue;
    const uint8_t sb = f32_to_e4m3(gmax[j] / (6.f * global));
    const float bs = e4m3_to_f32(sb);
    uint2 packed = make_uint2(0u, 0u);
    uint8_t scale_byte = 0;
    if (gmax[j] != 0.f && bs != 0.f) {
      scale_byte = sb;
      const float q = 1.f / (bs * global);
      uint32_t c[2] = {0u, 0u};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t lo = f32_to_e2m1(bits_f32(w[j][i] << 16) * q);
        const uint32_t hi = f32_to_e2m1(bits_f32(w[j][i] & 0xFFFF0000u) * q);
        c[i >> 2] |= (lo | (hi << 4)) << (8 * (i & 3));
      }
      packed = make_uint2(c[0], c[1]);
    }
    scale_row[g] = scale_byte;
    *reinterpret_cast<uint2*>(code_row + g * 8) = packed;
  }
}

template <int MODE, int RECIPE = 0>
hipError_t launch_quant(const QuantArgs& a, hipStream_t stream) {
  const int groups = a.k / 16;
  const int gpt = (groups + kQuantThreads - 1) / kQuantThreads;
  const dim3 grid(static_cast<unsigned>(a.rows)), block(kQuantThreads);
  if (gpt <= 1) hipLaunchKernelGGL((nvfp4_quantize_rows_kernel<1, MODE, RECIPE>), grid, block, 0, stream, a);
  else if (gpt <= 2) hipLaunchKernelGGL((nvfp4_quantize_rows_kernel<2, MODE, RECIPE>), grid, block, 0, stream, a);
  else if (gpt <= 4) hipLaunchKernelGGL((nvfp4_quantize_rows_kernel<4, MODE, RECIPE>), grid, block, 0, stream, a);
  else hipLaunchKernelGGL((nvfp4_quantize_rows_kernel<8, MODE, RECIPE>), grid, block, 0, stream, a);
  return hipGetLastError();
}

// SwiGLU of the native expert's first GEMM (src/kernels/minimax_native_moe.cu:87-95): FP32 gate / up sums ->
// bf16((g' / (1 + exp(-alpha g'))) (u' + 1)), g' = min(g, limit), u' = clamp(u, -limit, limit). Four values per lane.
__global__ __launch_bounds__(256) void swiglu_f32_rows_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                              uint16_t* __restrict__ out, int64_t count, float alpha,
                                                              float limit, int vec) {
  const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i0 >= count) return;
  auto one = [&](float gv, float uv) {
    const float g = fminf(gv, limit), u = fminf(fmaxf(uv, -limit), limit);
    return f32_to_bf16((g / (1.f + expf(-alpha * g))) * (u + 1.f));
  };
  if (vec && i0 + 4 <= count) {
    const float4 g = *reinterpret_cast<const float4*>(gate + i0), u = *reinterpret_cast<const float4*>(up + i0);
    const uint32_t lo = static_cast<uint32_t>(one(g.x, u.x)) | (static_cast<uint32_t>(one(g.y, u.y)) << 16);
    const uint32_t hi = static_cast<uint32_t>(one(g.z, u.z)) | (static_cast<uint32_t>(one(g.w, u.w)) << 16);
    *reinterpret_cast<uint2*>(out + i0) = make_uint2(lo, hi);
    return;
  }
  for (int64_t i = i0; i < count && i < i0 + 4; ++i) out[i] = one(gate[i], up[i]);
}

int quantize(const uint16_t* x, const uint16_t* up, size_t stride, int rows, int k, float limit, uint8_t* codes,
             uint8_t* scales, float* gs, void* stream, float static_gs, const float* static_gs_dev, int mode, const char* who) {
  if (rows <= 0) return DGPP_OK;
  if (k <= 0 || k % 64 != 0 || k > 32768) return report_invalid(std::string(who) + ": k must be a multiple of 64, <= 32768");
  if (!x || (mode != 0 && !up) || !codes || !scales || !gs) return report_invalid(std::string(who) + ": null pointer");
  if (stride % 8 != 0 || stride < static_cast<size_t>(k) || reinterpret_cast<uintptr_t>(x) % 16 != 0 ||
      (mode != 0 && reinterpret_cast<uintptr_t>(up) % 16 != 0))
    return report_invalid(std::string(who) + ": rows must be 16-byte aligned");
  if (reinterpret_cast<uintptr_t>(codes) % 8 != 0) return report_invalid(std::string(who) + ": codes must be 8-byte aligned");
  QuantArgs a;
  a.x = x;
  a.up = up;
  a.stride = stride;
  a.rows = rows;
  a.k = k;
  a.codes = codes;
  a.scales = scales;
  a.scale_stride = dgpp_nvfp4_act_scale_stride(k);
  a.gs = gs;
  a.static_gs = static_gs;
  a.static_gs_dev = static_gs_dev;
  a.limit = limit;
  a.aligned = 1;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const hipError_t err = mode == 0 ? launch_quant<0>(a, st) : (mode == 1 ? launch_quant<1>(a, st) : launch_quant<2>(a, st));
  return report_hip(err, who);
}

int grouped_w4a4(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                 const DgppMoeSegment* segs, int n_segs, int max_rows, const DgppMoeExpertView* views, int which, void* out,
                 int out_f32, size_t out_stride, int n, int k, void* stream) {
  const char* who = "moe w4a4";
  if (n_segs <= 0 || n <= 0) return DGPP_OK;
  if (k <= 0 || k % 64 != 0) return report_invalid(std::string(who) + ": k must be a multiple of 64");
  if (max_rows <= 0) return report_invalid(std::string(who) + ": max_rows");
  if (!codes || !scales || !gs || !segs || !views || !out) return report_invalid(std::string(who) + ": null pointer");
  if (which < 0 || which > 2) return report_invalid(std::string(who) + ": which must be 0, 1 or 2");
  if (out_stride < static_cast<size_t>(n)) return report_invalid(std::string(who) + ": out_stride below n");
  if (reinterpret_cast<uintptr_t>(codes) % 4 != 0) return report_invalid(std::string(who) + ": codes must be 4-byte aligned");
  const unsigned z_ext = 1u;
  if (n_segs > 65535) return report_invalid(std::string(who) + ": grid dimension overflow");
  GroupedArgs a;
  a.act = reinterpret_cast<const uint16_t*>(codes);
  a.act_stride = static_cast<size_t>(k) / 2;   // bytes per code row
  a.segs = segs;
  a.views = views;
  a.which = which;
  a.out = out;
  a.out_stride = out_stride;
  a.out_f32 = out_f32;
  a.n = n;
  a.k = k;
  a.rows_per_block = INT_MAX;
  a.group_rows = kMaxActRows;
  a.act_rows = act_rows;
  a.gate_up = 0;
  a.limit = 0.f;
  a.out_up = nullptr;
  a.once = max_rows <= kTileCols;
  a.a4_scales = scales;
  a.a4_scale_stride = dgpp_nvfp4_act_scale_stride(k);
  a.a4_gs = gs;
  return report_hip(launch_grouped_mma(kFmtNvfp4, a, n_segs, static_cast<int>(z_ext), static_cast<hipStream_t>(stream)), who);
}

int dense_w4a4(const uint8_t* a_codes, const uint8_t* a_scales, size_t a_scale_stride, const float* a_gs,
               const uint8_t* w_codes, const uint8_t* w_scales, const float* w_global, void* out, int out_f32, size_t out_stride,
               int m, int n, int k, void* stream) {
  const char* who = "dense w4a4";
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (k <= 0 || k % 128 != 0) return report_invalid(std::string(who) + ": k must be a multiple of 128");
  if (!a_codes || !a_scales || !a_gs || !w_codes || !w_scales || !w_global || !out)
    return report_invalid(std::string(who) + ": null pointer");
  if (out_stride < static_cast<size_t>(n)) return report_invalid(std::string(who) + ": out_stride below n");
  if (a_scale_stride < static_cast<size_t>(k / 16)) return report_invalid(std::string(who) + ": a_scale_stride below k / 16");
  if (reinterpret_cast<uintptr_t>(a_codes) % 16 != 0 || reinterpret_cast<uintptr_t>(w_codes) % 16 != 0)
    return report_invalid(std::string(who) + ": code matrices must be 16-byte aligned");
  if ((m + kTileCols - 1) / kTileCols > 65535) return report_invalid(std::string(who) + ": grid dimension overflow");
  DenseArgs a;
  a.act = reinterpret_cast<const uint16_t*>(a_codes);
  a.act_stride = static_cast<size_t>(k) / 2;   // bytes per code row
  a.mat.payload = w_codes;
  a.mat.scales = w_scales;
  a.mat.divisor = 1.f;
  a.mat.rs = 0;
  a.mat.cs = 0;
  a.global = w_global;
  a.out = out;
  a.out_stride = out_stride;
  a.out_f32 = out_f32;
  a.m = m;
  a.n = n;
  a.k = k;
  a.once = m <= kTileCols;
  a.a4_scales = a_scales;
  a.a4_scale_stride = a_scale_stride;
  a.a4_gs = a_gs;
  return report_hip(launch_dense_mma(kFmtNvfp4, a, nullptr, 0, static_cast<hipStream_t>(stream)), who);
}

}  // namespace
}  // namespace dgpp_amd

using namespace dgpp_amd;

extern "C" {

size_t dgpp_nvfp4_act_scale_stride(int k) { return static_cast<size_t>(((k / 16) + 7) / 8 * 8); }

int dgpp_minimax_quantize_rows_nvfp4(const uint16_t* input, size_t stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                     float* globals, void* stream) {
  const char* who = "minimax_quantize_rows_nvfp4";
  if (rows <= 0) return DGPP_OK;
  if (k <= 0 || k > 32768 || k % 128 != 0 || stride < static_cast<size_t>(k))
    return report_invalid(std::string(who) + ": k must be 128-aligned and <= 32768");
  if (!input || !codes || !scales || !globals) return report_invalid(std::string(who) + ": null pointer");
  if (reinterpret_cast<uintptr_t>(codes) % 8 != 0) return report_invalid(std::string(who) + ": codes must be 8-byte aligned");
  QuantArgs a{};
  a.x = input;
  a.stride = stride;
  a.rows = rows;
  a.k = k;
  a.codes = codes;
  a.scales = scales;
  a.scale_stride = static_cast<size_t>(k / 16);   // dense: no padding in this producer's layout
  a.gs = globals;
  a.aligned = stride % 8 == 0 && reinterpret_cast<uintptr_t>(input) % 16 == 0;
  return report_hip(launch_quant<0, 1>(a, static_cast<hipStream_t>(stream)), who);
}

int dgpp_minimax_swiglu_f32(const float* gate, const float* up, uint16_t* output, int64_t count, float alpha, float limit,
                            void* stream) {
  const char* who = "minimax_swiglu_f32";
  if (count <= 0) return DGPP_OK;
  if (!gate || !up || !output) return report_invalid(std::string(who) + ": null pointer");
  const int vec = ((reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up)) & 15u) == 0 &&
                  (reinterpret_cast<uintptr_t>(output) & 7u) == 0;
  const int64_t lanes = (count + 3) / 4;
  if ((lanes + 255) / 256 > 0x7FFFFFFFLL) return report_invalid(std::string(who) + ": grid dimension overflow");
  hipLaunchKernelGGL(swiglu_f32_rows_kernel, dim3(static_cast<unsigned>((lanes + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), gate, up, output, count, alpha, limit, vec);
  return report_hip(hipGetLastError(), who);
}

int dgpp_launch_quantize_rows_nvfp4(const uint16_t* x, size_t x_stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                    float* gs, void* stream, float static_gs, const float* static_gs_dev) {
  return quantize(x, nullptr, x_stride, rows, k, 0.f, codes, scales, gs, stream, static_gs, static_gs_dev, 0, "quantize nvfp4");
}

int dgpp_launch_swiglu_quantize_rows_nvfp4(const uint16_t* gate, const uint16_t* up, size_t stride, int rows, int k,
                                           float limit, uint8_t* codes, uint8_t* scales, float* gs, void* stream,
                                           float static_gs, const float* static_gs_dev, int qwen_rounding) {
  return quantize(gate, up, stride, rows, k, limit, codes, scales, gs, stream, static_gs, static_gs_dev, qwen_rounding ? 2 : 1,
                  "swiglu quantize nvfp4");
}

int dgpp_launch_moe_grouped_w4a4_bf16(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                                      const DgppMoeSegment* segs, int n_segs, int max_rows, const DgppMoeExpertView* views,
                                      int which, uint16_t* out, size_t out_stride, int n, int k, void* stream) {
  return grouped_w4a4(codes, scales, gs, act_rows, segs, n_segs, max_rows, views, which, out, 0, out_stride, n, k, stream);
}

int dgpp_launch_moe_grouped_w4a4_f32(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                                     const DgppMoeSegment* segs, int n_segs, int max_rows, const DgppMoeExpertView* views,
                                     int which, float* out, size_t out_stride, int n, int k, void* stream) {
  return grouped_w4a4(codes, scales, gs, act_rows, segs, n_segs, max_rows, views, which, out, 1, out_stride, n, k, stream);
}

int dgpp_dense_w4a4_supported(int k) { return k > 0 && k % 128 == 0; }

int dgpp_launch_dense_w4a4_bf16(const uint8_t* a_codes, const uint8_t* a_scales, size_t a_scale_stride, const float* a_gs,
                                const uint8_t* w_codes, const uint8_t* w_scales, const float* w_global, uint16_t* out,
                                size_t out_stride, int m, int n, int k, void* stream) {
  return dense_w4a4(a_codes, a_scales, a_scale_stride, a_gs, w_codes, w_scales, w_global, out, 0, out_stride, m, n, k, stream);
}

}  // extern "C"
