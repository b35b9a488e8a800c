// Activation-quantized MXFP8 form: per-row dynamic MXFP8 quantizers (plain, and fused behind the
// clamped SwiGLU of the MiniMax shared expert) and the block-scaled E4M3 x E4M3 GEMM on the
// scaled matrix-core instruction V_MFMA_SCALE_F32_16X16X128_F8F6F4, which takes both payloads as
// stored and one e8m0 scale per 32 values of either operand: no weight decode on the VALU at all.
//
// Reference counterparts: src/kernels/mxfp8_gemm.hpp:8-31 (interface), src/kernels/mxfp8_gemm.cu:24-79
// (quantizer), :106-203 (GEMM), :217-243 (argument rules), :246-275 (launchers).
#include <hip/hip_runtime.h>

#include <string>

#include "../../include/dgpp_amd.h"
#include "capi_errors.hpp"
#include "numerics.hpp"

namespace dgpp_amd {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kQuantThreads = 256;
constexpr int kGemmWaves = 4;
constexpr int kGemmThreads = kGemmWaves * 64;

// ---- quantizers ----------------------------------------------------------------------------------

// The e8m0 exponent of a 32-group whose largest magnitude is `maximum`: ceil(log2(maximum / 448)), at
// least -127, read off the float's own fields (448 = 1.75 * 2^8, so the ceiling steps where the
// significand passes 1.75). src/kernels/mxfp8_gemm.cu:61-66.
__device__ __forceinline__ int group_exponent(float maximum) {
  const int biased = static_cast<int>((f32_bits(maximum) >> 23) & 255u);
  const float threshold = bits_f32((static_cast<uint32_t>(biased) << 23) | 0x600000u);
  const int e = biased - 135 + (maximum > threshold ? 1 : 0);
  return e < -127 ? -127 : e;
}

// Four E4M3 codes (round to nearest even; the scaled group never exceeds 448, the clamp only keeps an
// out-of-contract input finite) in one word, lowest address first.
__device__ __forceinline__ uint32_t pack_e4m3x4(float v0, float v1, float v2, float v3) {
  v0 = __builtin_amdgcn_fmed3f(v0, -448.f, 448.f);
  v1 = __builtin_amdgcn_fmed3f(v1, -448.f, 448.f);
  v2 = __builtin_amdgcn_fmed3f(v2, -448.f, 448.f);
  v3 = __builtin_amdgcn_fmed3f(v3, -448.f, 448.f);
  int word = 0;
  word = __builtin_amdgcn_cvt_pk_fp8_f32(v0, v1, word, false);
  word = __builtin_amdgcn_cvt_pk_fp8_f32(v2, v3, word, true);
  return static_cast<uint32_t>(word);
}

__device__ __forceinline__ void unpack_bf16x4(const uint2& q, float (&v)[4]) {
  v[0] = bits_f32(q.x << 16);
  v[1] = bits_f32(q.x & 0xffff0000u);
  v[2] = bits_f32(q.y << 16);
  v[3] = bits_f32(q.y & 0xffff0000u);
}

// One lane holds four adjacent values, eight lanes one 32-group (rows may start on any multiple of four
// elements, as in the reference). A row is k / 4 lanes; blockIdx.y is the row. With SWIGLU the values
// are first bf16(min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, +-limit) + 1)), the sigmoid
// through the hardware's base-2 exponential and reciprocal where the reference goes through its
// approximate ones (src/kernels/mxfp8_gemm.cu:37-56).
template <bool SWIGLU>
__global__ __launch_bounds__(kQuantThreads) void mxfp8_quantize_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ up, size_t stride, int k, float alpha, float limit,
    uint8_t* __restrict__ codes, uint8_t* __restrict__ scales) {
  const int row = blockIdx.y;
  const int piece = blockIdx.x * kQuantThreads + threadIdx.x;
  const int column = piece * 4;
  // k is a multiple of 32, so the eight lanes of a group leave together.
  if (column >= k) return;
  float v[4];
  unpack_bf16x4(*reinterpret_cast<const uint2*>(x + static_cast<size_t>(row) * stride + column), v);
  if constexpr (SWIGLU) {
    float u[4];
    unpack_bf16x4(*reinterpret_cast<const uint2*>(up + static_cast<size_t>(row) * stride + column), u);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float g = fminf(v[i], limit);
      const float uc = fminf(fmaxf(u[i], -limit), limit);
      const float e = __builtin_amdgcn_exp2f((g * -alpha) * 1.4426950216293335f);
      const float sigmoid = __builtin_amdgcn_rcpf(1.f + e);
      v[i] = bf16_to_f32(f32_to_bf16((g * sigmoid) * (uc + 1.f)));
    }
  }
  float maximum = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
  maximum = fmaxf(maximum, __shfl_xor(maximum, 1));
  maximum = fmaxf(maximum, __shfl_xor(maximum, 2));
  maximum = fmaxf(maximum, __shfl_xor(maximum, 4));
  const int exponent = group_exponent(maximum);
  const float inverse = bits_f32(static_cast<uint32_t>(127 - exponent) << 23);
  *reinterpret_cast<uint32_t*>(codes + static_cast<size_t>(row) * k + column) =
      pack_e4m3x4(v[0] * inverse, v[1] * inverse, v[2] * inverse, v[3] * inverse);
  if ((piece & 7) == 0) scales[static_cast<size_t>(row) * (k >> 5) + (column >> 5)] = static_cast<uint8_t>(exponent + 127);
}

// ---- GEMM ----------------------------------------------------------------------------------------

__device__ __forceinline__ v8i as_operand(const u32x4& lo, const u32x4& hi) {
  v8i r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i] = static_cast<int>(lo[i]);
    r[4 + i] = static_cast<int>(hi[i]);
  }
  return r;
}

template <typename Out>
__device__ __forceinline__ void put(Out* p, float v);
template <>
__device__ __forceinline__ void put<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void put<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

// out[m, n] = A[m, k] * W[n, k]^T. A block owns 16 rows of W over all of k and MT * 16 rows of A.
//
// One matrix-core step covers 128 of k. Lane (r, g) = (lane % 16, lane / 16) hands over, for row r of
// its 16, the 16 bytes at k = 16 g of the step in the operand's registers 0-3 and the 16 bytes at
// k = 64 + 16 g in registers 4-7 (so one load instruction of the wave reads 64 contiguous bytes of each
// of the 16 rows), and the scale byte of the row's k-block g of the step, which the hardware applies to
// that block wherever its bytes sit (block b of a row is held by lanes 2 (b % 2) and 2 (b % 2) + 1, in
// registers 4 (b / 2) .. 4 (b / 2) + 3). W is the first operand, a 16-row tile of A the second; the lane
// receives out[a row r][w rows 4 g .. 4 g + 3].
// The block's four waves take the steps in pairs, wave w the pairs w, w + 4, ...; their partial sums
// are added in wave order by wave 0. The chain of every output element is therefore fixed by k alone,
// whatever m, n and the rows that share a launch (src/kernels/mxfp8_gemm.hpp:23 asks the same of the
// reference's row geometries).
// Rows past n or m are clamped to the last one and never stored; bytes past k contribute zeros.
template <typename Out, int MT>
__global__ __launch_bounds__(kGemmThreads) void mxfp8_gemm_kernel(
    const uint8_t* __restrict__ a, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ w,
    const uint8_t* __restrict__ w_scales, Out* __restrict__ out, int m, int n, int k, size_t out_stride) {
  __shared__ float4 fold[kGemmWaves - 1][MT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * (16 * MT);
  const int kblocks = k >> 5;
  const int steps = (kblocks + 3) >> 2;

  const int w_row = min(n0 + r, n - 1);
  const uint8_t* wp = w + static_cast<size_t>(w_row) * k;
  const uint8_t* wsp = w_scales + static_cast<size_t>(w_row) * kblocks;
  const uint8_t* ap[MT];
  const uint8_t* asp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int a_row = min(m0 + t * 16 + r, m - 1);
    ap[t] = a + static_cast<size_t>(a_row) * k;
    asp[t] = a_scales + static_cast<size_t>(a_row) * kblocks;
  }

  v4f acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int s = wave * 2; s < steps; s += kGemmWaves * 2) {
    u32x4 wq[2][2], aq[2][MT][2];
    int ws[2], as[2][MT];
    bool valid[2][2];
    // Every load of the pair is issued before the first use.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int kb = (s + j) * 4 + g;
      const int kc = kb < kblocks ? kb : kblocks - 1;
      ws[j] = wsp[kc];
#pragma unroll
      for (int t = 0; t < MT; ++t) as[j][t] = asp[t][kc];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int at = (s + j) * 128 + h * 64 + g * 16;
        valid[j][h] = at < k;
        const int off = valid[j][h] ? at : 0;
        wq[j][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + off));
#pragma unroll
        for (int t = 0; t < MT; ++t) aq[j][t][h] = *reinterpret_cast<const u32x4*>(ap[t] + off);
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
        if (!valid[j][h]) {
          wq[j][h] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int t = 0; t < MT; ++t) aq[j][t][h] = u32x4{0u, 0u, 0u, 0u};
        }
      const v8i wv = as_operand(wq[j][0], wq[j][1]);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, as_operand(aq[j][t][0], aq[j][t][1]), acc[t],
                                                                  0, 0, 0, ws[j], 0, as[j][t]);
    }
  }

  if (wave != 0) {
#pragma unroll
    for (int t = 0; t < MT; ++t) fold[wave - 1][t][lane] = float4{acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    float sum[4] = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
#pragma unroll
    for (int p = 0; p < kGemmWaves - 1; ++p) {
      const float4 part = fold[p][t][lane];
      sum[0] += part.x;
      sum[1] += part.y;
      sum[2] += part.z;
      sum[3] += part.w;
    }
    const int a_row = m0 + t * 16 + r;
    if (a_row >= m) continue;
    Out* dst = out + static_cast<size_t>(a_row) * out_stride + n0 + g * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n0 + g * 4 + i < n) put<Out>(dst + i, sum[i]);
  }
}

template <typename Out, int MT>
hipError_t launch_gemm_mt(const uint8_t* a, const uint8_t* as, const uint8_t* w, const uint8_t* ws, Out* out, int m, int n,
                          int k, size_t stride, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((n + 15) / 16), static_cast<unsigned>((m + 16 * MT - 1) / (16 * MT)));
  hipLaunchKernelGGL((mxfp8_gemm_kernel<Out, MT>), grid, dim3(kGemmThreads), 0, stream, a, as, w, ws, out, m, n, k, stride);
  return hipGetLastError();
}

// src/kernels/mxfp8_gemm.cu:217-243.
template <typename Out>
int gemm(const uint8_t* a, const uint8_t* as, const uint8_t* w, const uint8_t* ws, Out* out, int m, int n, int k,
         void* stream, size_t stride, int output_tile) {
  const char* who = "MXFP8 GEMM";
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (k <= 0 || k % 64) return report_invalid(std::string(who) + ": k must be a positive multiple of 64");
  if (stride == 0) stride = static_cast<size_t>(n);
  if (stride < static_cast<size_t>(n)) return report_invalid(std::string(who) + ": output stride is too small");
  if (output_tile != 0 && output_tile != 8 && output_tile != 16 && output_tile != 32 && output_tile != 64)
    return report_invalid(std::string(who) + ": output tile must be 0, 8, 16, 32 or 64");
  if (!a || !as || !w || !ws || !out) return report_invalid(std::string(who) + ": null pointer");
  if (((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) & 15u) != 0)
    return report_invalid(std::string(who) + ": payloads must be 16-byte aligned");
  // The tile override is a diagnostic of the reference's kernel; every value gives the same chain here.
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t err;
  if (m <= 16)
    err = launch_gemm_mt<Out, 1>(a, as, w, ws, out, m, n, k, stride, s);
  else if (m <= 32)
    err = launch_gemm_mt<Out, 2>(a, as, w, ws, out, m, n, k, stride, s);
  else if (m <= 48)
    err = launch_gemm_mt<Out, 3>(a, as, w, ws, out, m, n, k, stride, s);
  else
    err = launch_gemm_mt<Out, 4>(a, as, w, ws, out, m, n, k, stride, s);
  return report_hip(err, who);
}

// src/kernels/mxfp8_gemm.cu:246-268. A lane reads 8 bytes and writes 4, so besides the reference's rules
// (32-wide groups, a stride of at least k and a multiple of four elements) the rows start 8-byte aligned.
int quantize(const uint16_t* x, const uint16_t* up, bool fused, size_t stride, int rows, int k, float alpha, float limit,
             uint8_t* codes, uint8_t* scales, void* stream, const char* who) {
  if (rows <= 0) return DGPP_OK;
  if (k <= 0 || k % 32 || stride < static_cast<size_t>(k) || stride % 4)
    return report_invalid(std::string(who) + ": requires 32-wide groups and aligned input rows");
  if (!x || !codes || !scales || (fused && !up)) return report_invalid(std::string(who) + ": null pointer");
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(up)) & 7u) != 0 ||
      (reinterpret_cast<uintptr_t>(codes) & 3u) != 0)
    return report_invalid(std::string(who) + ": input rows must be 8-byte aligned, codes 4-byte aligned");
  if (rows > 65535) return report_invalid(std::string(who) + ": more than 65535 rows");
  const dim3 grid(static_cast<unsigned>((k / 4 + kQuantThreads - 1) / kQuantThreads), static_cast<unsigned>(rows));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (fused)
    hipLaunchKernelGGL((mxfp8_quantize_kernel<true>), grid, dim3(kQuantThreads), 0, s, x, up, stride, k, alpha, limit, codes, scales);
  else
    hipLaunchKernelGGL((mxfp8_quantize_kernel<false>), grid, dim3(kQuantThreads), 0, s, x, up, stride, k, 0.f, 0.f, codes, scales);
  return report_hip(hipGetLastError(), who);
}

}  // namespace
}  // namespace dgpp_amd

using namespace dgpp_amd;

extern "C" {

int dgpp_launch_mxfp8_quantize_rows(const uint16_t* x, size_t x_stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                    void* stream) {
  return quantize(x, nullptr, false, x_stride, rows, k, 0.f, 0.f, codes, scales, stream, "MXFP8 quantize");
}
int dgpp_launch_minimax_swiglu_mxfp8_rows(const uint16_t* gate, const uint16_t* up, size_t stride, int rows, int k, float alpha,
                                          float limit, uint8_t* codes, uint8_t* scales, void* stream) {
  return quantize(gate, up, true, stride, rows, k, alpha, limit, codes, scales, stream, "MiniMax SwiGLU MXFP8");
}
int dgpp_launch_mxfp8_gemm_bf16(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales,
                                uint16_t* out, int m, int n, int k, void* stream, size_t out_stride, int output_tile) {
  return gemm<uint16_t>(a, a_scales, w, w_scales, out, m, n, k, stream, out_stride, output_tile);
}
int dgpp_launch_mxfp8_gemm_f32(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales, float* out,
                               int m, int n, int k, void* stream, size_t out_stride, int output_tile) {
  return gemm<float>(a, a_scales, w, w_scales, out, m, n, k, stream, out_stride, output_tile);
}

}  // extern "C"
