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
// One matrix-core step covers 128 of k. Its operand layout: lane (r, g) = (lane % 16, lane / 16) holds,
// for row r of its 16, the 16 bytes at k = 16 g of the step in registers 0-3 and the 16 bytes at
// k = 64 + 16 g in registers 4-7, and supplies the scale byte of the row's k-block g of the step, which
// the hardware applies to that block wherever its bytes sit. W is the first operand, a 16-row tile of A
// the second; the lane receives out[a row r][w rows 4 g .. 4 g + 3].
//
// Loading in that layout would ask the memory pipe for 64 bytes of 16 different rows per instruction,
// which it serves at about half its streaming rate. A step's 16 x 128 bytes of either operand are
// therefore loaded row-major (two instructions of 8 rows x 128 contiguous bytes), parked in a
// wavefront-private LDS region and read back in operand layout; the region is XOR-swizzled so that the
// writes and the reads both touch every bank once.
//
// The block's WAVES waves split k: wave w takes the steps w, w + WAVES, ..., and the partial sums are
// added in wave order (tile t by wave t). The chain of every output element is therefore fixed by k alone
// (WAVES is chosen from k), whatever m, n and the rows that share a launch
// (src/kernels/mxfp8_gemm.hpp:23 asks the same of the reference's row geometries).
// Rows past n or m are clamped to the last one and never stored; bytes past k contribute zeros.
constexpr int kStepUnits = 128;   // 16-byte units of one step of one operand tile: 16 rows x 128 bytes

// The swizzled place of 16-byte piece `piece` (0-7) of row `row` (0-15) in a region.
__device__ __forceinline__ int region_unit(int row, int piece) { return row * 8 + (piece ^ ((row >> 1) & 7)); }

// This lane's two row-major loads of a step: rows (lane / 8) and 8 + (lane / 8) of the 16 that start at
// row0 (clamped to the last row), piece lane % 8 of the step's 128 bytes; zeros past k.
template <bool NT>
__device__ __forceinline__ void issue_step(const uint8_t* __restrict__ base, int row0, int rows, int k, int step,
                                           u32x4 (&t)[2]) {
  const int lane = threadIdx.x & 63;
  const int at = step * 128 + (lane & 7) * 16;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = min(row0 + 8 * i + (lane >> 3), rows - 1);
    const u32x4* src = reinterpret_cast<const u32x4*>(base + static_cast<size_t>(row) * k + (at < k ? at : 0));
    const u32x4 v = NT ? __builtin_nontemporal_load(src) : *src;
    t[i] = at < k ? v : u32x4{0u, 0u, 0u, 0u};
  }
}
__device__ __forceinline__ void commit_step(u32x4* __restrict__ region, const u32x4 (&t)[2]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < 2; ++i) region[region_unit(8 * i + (lane >> 3), lane & 7)] = t[i];
}
__device__ __forceinline__ v8i step_operand(const u32x4* __restrict__ region) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  return as_operand(region[region_unit(r, g)], region[region_unit(r, 4 + g)]);
}

template <typename Out, int MT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void mxfp8_gemm_kernel(
    const uint8_t* __restrict__ a, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ w,
    const uint8_t* __restrict__ w_scales, Out* __restrict__ out, int m, int n, int k, size_t out_stride) {
  static_assert(WAVES >= MT, "one folding wave per tile");
  // Two regions per wave while the steps run, the partial sums of every wave afterwards.
  constexpr int kStageUnits = WAVES * 2 * kStepUnits, kFoldUnits = WAVES * MT * 64;
  __shared__ u32x4 lds[kStageUnits > kFoldUnits ? kStageUnits : kFoldUnits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * (16 * MT);
  const int kblocks = k >> 5;
  const int steps = (kblocks + 3) >> 2;
  u32x4* region = lds + wave * 2 * kStepUnits;

  const uint8_t* wsp = w_scales + static_cast<size_t>(min(n0 + r, n - 1)) * kblocks;
  const uint8_t* asp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) asp[t] = a_scales + static_cast<size_t>(min(m0 + t * 16 + r, m - 1)) * kblocks;

  v4f acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};

  // Steps interleave over the waves, so that at any time the block reads a few KB of each row in one piece.
  // DEPTH steps of a wave are in flight together: every load of them is issued before the first use.
  constexpr int DEPTH = MT == 1 ? 4 : MT == 2 ? 2 : 1;
  for (int s0 = wave; s0 < steps; s0 += WAVES * DEPTH) {
    u32x4 wq[DEPTH][2], aq[DEPTH][MT][2];
    int ws[DEPTH], as[DEPTH][MT];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int s = s0 + d * WAVES;
      if (s >= steps) break;   // the same for the whole wave
      issue_step<true>(w, n0, n, k, s, wq[d]);
#pragma unroll
      for (int t = 0; t < MT; ++t) issue_step<false>(a, m0 + t * 16, m, k, s, aq[d][t]);
      const int kb = s * 4 + g;
      const int kc = kb < kblocks ? kb : kblocks - 1;   // a block past k holds zeros: any scale does
      ws[d] = wsp[kc];
#pragma unroll
      for (int t = 0; t < MT; ++t) as[d][t] = asp[t][kc];
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (s0 + d * WAVES >= steps) break;
      // The LDS serves a wavefront's accesses in order: a region is rewritten as soon as the read of its
      // previous content has been issued. The barriers only keep the compiler from moving accesses across.
      commit_step(region, wq[d]);
      __builtin_amdgcn_wave_barrier();
      const v8i wv = step_operand(region);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        u32x4* mine = region + ((t + 1) & 1) * kStepUnits;   // the other region than the tile before
        commit_step(mine, aq[d][t]);
        __builtin_amdgcn_wave_barrier();
        acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, step_operand(mine), acc[t], 0, 0, 0, ws[d], 0, as[d][t]);
      }
    }
  }

  __syncthreads();   // every wave is done with its regions
  float4* fold = reinterpret_cast<float4*>(lds);
#pragma unroll
  for (int t = 0; t < MT; ++t) fold[(wave * MT + t) * 64 + lane] = float4{acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
  __syncthreads();
  if (wave >= MT) return;
  const int t = wave;
  float4 sum = fold[t * 64 + lane];
#pragma unroll
  for (int p = 1; p < WAVES; ++p) {
    const float4 part = fold[(p * MT + t) * 64 + lane];
    sum.x += part.x;
    sum.y += part.y;
    sum.z += part.z;
    sum.w += part.w;
  }
  const int a_row = m0 + t * 16 + r;
  if (a_row >= m) return;
  Out* dst = out + static_cast<size_t>(a_row) * out_stride + n0 + g * 4;
  const float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (n0 + g * 4 + i < n) put<Out>(dst + i, v[i]);
}

template <typename Out, int MT, int WAVES>
hipError_t launch_gemm_mt(const uint8_t* a, const uint8_t* as, const uint8_t* w, const uint8_t* ws, Out* out, int m, int n,
                          int k, size_t stride, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((n + 15) / 16), static_cast<unsigned>((m + 16 * MT - 1) / (16 * MT)));
  hipLaunchKernelGGL((mxfp8_gemm_kernel<Out, MT, WAVES>), grid, dim3(WAVES * 64), 0, stream, a, as, w, ws, out, m, n, k, stride);
  return hipGetLastError();
}

template <typename Out, int WAVES>
hipError_t launch_gemm_waves(const uint8_t* a, const uint8_t* as, const uint8_t* w, const uint8_t* ws, Out* out, int m, int n,
                             int k, size_t stride, hipStream_t s) {
  if (m <= 16) return launch_gemm_mt<Out, 1, WAVES>(a, as, w, ws, out, m, n, k, stride, s);
  if (m <= 32) return launch_gemm_mt<Out, 2, WAVES>(a, as, w, ws, out, m, n, k, stride, s);
  if (m <= 48) return launch_gemm_mt<Out, 3, WAVES>(a, as, w, ws, out, m, n, k, stride, s);
  return launch_gemm_mt<Out, 4, WAVES>(a, as, w, ws, out, m, n, k, stride, s);
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
  // Waves per block from k alone (an output element's chain must not depend on m or n): sixteen once every
  // wave has a step of its own.
  hipStream_t s = static_cast<hipStream_t>(stream);
  const hipError_t err = k >= 16 * 128 ? launch_gemm_waves<Out, 16>(a, as, w, ws, out, m, n, k, stride, s)
                                       : launch_gemm_waves<Out, 4>(a, as, w, ws, out, m, n, k, stride, s);
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
