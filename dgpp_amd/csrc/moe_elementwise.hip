// Elementwise and accumulation kernels of the MoE path: SwiGLU on finished gate / up rows, the row gather, the
// weighted accumulation back to tokens in its three forms (slot layout, grouped layout, scatter), the final bf16
// rounding, the FP8 -> BF16 bridge and the streaming probes of the measurement harness.
//
// These kernels move a few hundred KB to a few MB and are latency-bound: every lane works on 16 bytes (four fp32
// or eight bf16 values), a token's chain set-up (which rows, which weights, in which order) is computed ONCE per
// wavefront by lane operations and broadcast from lanes to scalar registers, and all rows of a chain are loaded
// before the first fma so that one trip to memory covers the chain.
//
// Arithmetic contracts (reference: src/kernels/glm_moe.cu:331-347 SwiGLU, :371-393 scatter / round, :673-711 slot
// chain, :1446-1489 ordered chain; src/kernels/fp8_dequant.cu:33-50): a chain is a = 0; a = fma(w_j, y_j, a) in the
// stated order, the shared row last with weight 1, one rounding to bf16 (or none).
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"
#include "moe_misc.hpp"
#include "numerics.hpp"
#include "swiglu.hpp"

namespace dgpp_amd {
namespace {

constexpr int kWaveLanes = 64;
constexpr int kFlatThreads = 256;

__device__ __forceinline__ bool aligned_to(const void* p, unsigned bytes) {
  return (reinterpret_cast<uintptr_t>(p) & (bytes - 1u)) == 0;
}
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}
__device__ __forceinline__ int lane_i32(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float lane_f32(float v, int lane) {
  return bits_f32(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(f32_bits(v)), lane)));
}

// ---- SwiGLU over flat [n] gate / up values, eight per lane -------------------------------------------------------
__global__ __launch_bounds__(kFlatThreads) void swiglu_flat_kernel(const uint16_t* __restrict__ gate,
                                                                   const uint16_t* __restrict__ up,
                                                                   uint16_t* __restrict__ out, int64_t n, float limit,
                                                                   int vec) {
  const int64_t e0 = (static_cast<int64_t>(blockIdx.x) * kFlatThreads + threadIdx.x) * 8;
  if (e0 >= n) return;
  if (vec && e0 + 8 <= n) {
    const uint4 g = *reinterpret_cast<const uint4*>(gate + e0);
    const uint4 u = *reinterpret_cast<const uint4*>(up + e0);
    *reinterpret_cast<uint4*>(out + e0) = swiglu_bf16x8(g, u, limit);
    return;
  }
  for (int64_t e = e0; e < n && e < e0 + 8; ++e) out[e] = swiglu_bf16(bf16_to_f32(gate[e]), bf16_to_f32(up[e]), limit);
}

// ---- row gather ----------------------------------------------------------------------------------------------------
__global__ void gather_rows_kernel(const uint16_t* __restrict__ src, const int32_t* __restrict__ rows,
                                   uint16_t* __restrict__ dst, int64_t n_units, int units_per_row, int unit_elems,
                                   int hidden) {
  // A unit is 8 elements (16 bytes) when rows allow vector copies, else one element.
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n_units) return;
  const int64_t r = i / units_per_row;
  const int64_t c = (i - r * units_per_row) * unit_elems;
  const uint16_t* s = src + static_cast<int64_t>(rows[r]) * hidden + c;
  uint16_t* d = dst + r * hidden + c;
  if (unit_elems == 8)
    *reinterpret_cast<uint4*>(d) = *reinterpret_cast<const uint4*>(s);
  else
    *d = *s;
}

// ---- scatter accumulation: acc[rows[r], :] = fma(w[r], y[r, :], acc[rows[r], :]) ---------------------------------------
// grid (source rows, column tiles of 4 * kFlatThreads); rows[] must not repeat a target row inside one launch.
template <bool VEC>
__global__ __launch_bounds__(kFlatThreads) void scatter_fma_kernel(float* __restrict__ acc, const float* __restrict__ y,
                                                                   const int32_t* __restrict__ rows,
                                                                   const float* __restrict__ row_w, int hidden) {
  const int r = static_cast<int>(blockIdx.x);
  const int col = (static_cast<int>(blockIdx.y) * kFlatThreads + static_cast<int>(threadIdx.x)) * 4;
  if (col >= hidden) return;
  const float w = row_w[r];
  float* d = acc + static_cast<size_t>(rows[r]) * hidden + col;
  const float* s = y + static_cast<size_t>(r) * hidden + col;
  if constexpr (VEC) {
    const float4 a = *reinterpret_cast<const float4*>(d), v = *reinterpret_cast<const float4*>(s);
    *reinterpret_cast<float4*>(d) = make_float4(fmaf(w, v.x, a.x), fmaf(w, v.y, a.y), fmaf(w, v.z, a.z), fmaf(w, v.w, a.w));
  } else {
    for (int i = 0; i < 4 && col + i < hidden; ++i) d[i] = fmaf(w, s[i], d[i]);
  }
}

// ---- bf16 rounding of a flat fp32 buffer, eight per lane ---------------------------------------------------------------
__global__ __launch_bounds__(kFlatThreads) void round_flat_kernel(uint16_t* __restrict__ out, const float* __restrict__ acc,
                                                                  int64_t n, int vec) {
  const int64_t e0 = (static_cast<int64_t>(blockIdx.x) * kFlatThreads + threadIdx.x) * 8;
  if (e0 >= n) return;
  if (vec && e0 + 8 <= n) {
    const float4 a = *reinterpret_cast<const float4*>(acc + e0), b = *reinterpret_cast<const float4*>(acc + e0 + 4);
    *reinterpret_cast<uint4*>(out + e0) =
        make_uint4(pack2_bf16(a.x, a.y), pack2_bf16(a.z, a.w), pack2_bf16(b.x, b.y), pack2_bf16(b.z, b.w));
    return;
  }
  for (int64_t e = e0; e < n && e < e0 + 8; ++e) out[e] = f32_to_bf16(acc[e]);
}

// ---- a token's accumulation chain ---------------------------------------------------------------------------------------
// One wavefront per (token, 256 columns), four adjacent columns per lane. The chain's K (row, weight) pairs are
// set up by lanes 0 .. K-1 and handed to every lane through scalar registers:
//   slot layout    row j = t * (K + 1) + j, weight weights[t, j]; `shared` adds row t * (K + 1) + K last
//   grouped layout the token's slots in ascending expert id (ties keep slot order): lane j ranks its id among the K
//                  with K lane reads, lane p then takes over the slot of rank p; row = slot_row[slot], weight
//                  slot_w[slot]; shared_row0 >= 0 adds row shared_row0 + t last
struct ChainArgs {
  void* out;
  const float* src;
  size_t src_stride;
  const int32_t* slot_row;   // grouped layout only
  const int32_t* slot_ids;   // grouped layout only
  const float* weights;      // [tokens, K]
  int shared;                // slot layout: 0 / 1; grouped layout: shared_row0 (< 0: none)
  int K, hidden;
  int src_bf16 = 0;          // the rows at `src` are BF16 (stride in BF16 elements), widened exactly as they are read
};

template <int KMAX, bool VEC, bool GROUPED, bool F32>
__global__ __launch_bounds__(kWaveLanes) void token_chain_kernel(ChainArgs a) {
  const int t = static_cast<int>(blockIdx.x), lane = static_cast<int>(threadIdx.x);
  const int col = (static_cast<int>(blockIdx.y) * kWaveLanes + lane) * 4;
  const int K = a.K;
  int my_row = 0;
  float my_w = 0.f;
  int shared_row = -1;
  if constexpr (GROUPED) {
    const int id = lane < K ? a.slot_ids[static_cast<size_t>(t) * K + lane] : INT_MAX;
    int rank = 0;
    for (int i = 0; i < K; ++i) {
      const int other = lane_i32(id, i);
      rank += (other < id) || (other == id && i < lane);
    }
    int from = 0;   // the slot whose rank is this lane's index
    for (int i = 0; i < K; ++i) from = lane_i32(rank, i) == lane ? i : from;
    if (lane < K) {
      const size_t s = static_cast<size_t>(t) * K + from;
      my_row = a.slot_row[s];
      my_w = a.weights[s];
    }
    if (a.shared >= 0) shared_row = a.shared + t;
  } else {
    if (lane < K) {
      my_row = t * (K + 1) + lane;
      my_w = a.weights[static_cast<size_t>(t) * K + lane];
    }
    if (a.shared) shared_row = t * (K + 1) + K;
  }
  const bool live = col < a.hidden;
  float v[KMAX + 1][4];
  auto fetch = [&](int row, float (&dst)[4]) {
    if (a.src_bf16) {
      const uint16_t* h = reinterpret_cast<const uint16_t*>(a.src) + static_cast<size_t>(row) * a.src_stride + col;
      if constexpr (VEC) {
        const uint2 q = live ? *reinterpret_cast<const uint2*>(h) : make_uint2(0u, 0u);
        dst[0] = bits_f32(q.x << 16), dst[1] = bits_f32(q.x & 0xFFFF0000u);
        dst[2] = bits_f32(q.y << 16), dst[3] = bits_f32(q.y & 0xFFFF0000u);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = col + i < a.hidden ? bf16_to_f32(h[i]) : 0.f;
      }
      return;
    }
    const float* p = a.src + static_cast<size_t>(row) * a.src_stride + col;
    if constexpr (VEC) {
      const float4 q = live ? *reinterpret_cast<const float4*>(p) : make_float4(0.f, 0.f, 0.f, 0.f);
      dst[0] = q.x, dst[1] = q.y, dst[2] = q.z, dst[3] = q.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[i] = col + i < a.hidden ? p[i] : 0.f;
    }
  };
#pragma unroll
  for (int j = 0; j < KMAX; ++j)
    if (j < K) fetch(lane_i32(my_row, j), v[j]);
  if (shared_row >= 0) fetch(shared_row, v[KMAX]);
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    if (j < K) {
      const float w = lane_f32(my_w, j);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(w, v[j][i], acc[i]);
    }
  }
  if (shared_row >= 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(1.0f, v[KMAX][i], acc[i]);
  }
  if (!live) return;
  const size_t at = static_cast<size_t>(t) * a.hidden + col;
  if constexpr (F32) {
    float* o = static_cast<float*>(a.out) + at;
    if constexpr (VEC) {
      *reinterpret_cast<float4*>(o) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    } else {
      for (int i = 0; i < 4 && col + i < a.hidden; ++i) o[i] = acc[i];
    }
  } else {
    uint16_t* o = static_cast<uint16_t*>(a.out) + at;
    if constexpr (VEC) {
      *reinterpret_cast<uint2*>(o) = make_uint2(pack2_bf16(acc[0], acc[1]), pack2_bf16(acc[2], acc[3]));
    } else {
      for (int i = 0; i < 4 && col + i < a.hidden; ++i) o[i] = f32_to_bf16(acc[i]);
    }
  }
}

template <bool GROUPED>
hipError_t launch_chain(const ChainArgs& a, int out_f32, int tokens, hipStream_t stream) {
  if (tokens <= 0 || a.hidden <= 0) return hipSuccess;
  const bool vec = a.hidden % 4 == 0 && a.src_stride % 4 == 0 &&
                   (reinterpret_cast<uintptr_t>(a.src) & (a.src_bf16 ? 7u : 15u)) == 0 &&
                   (reinterpret_cast<uintptr_t>(a.out) & (out_f32 ? 15u : 7u)) == 0;
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>((a.hidden + 4 * kWaveLanes - 1) / (4 * kWaveLanes)));
  auto go = [&](auto kmax, auto vc, auto fc) {
    hipLaunchKernelGGL((token_chain_kernel<decltype(kmax)::value, decltype(vc)::value, GROUPED, decltype(fc)::value>), grid,
                       dim3(kWaveLanes), 0, stream, a);
  };
  auto pick_f = [&](auto kmax, auto vc) {
    if (out_f32) go(kmax, vc, std::true_type{});
    else go(kmax, vc, std::false_type{});
  };
  auto pick_v = [&](auto kmax) {
    if (vec) pick_f(kmax, std::true_type{});
    else pick_f(kmax, std::false_type{});
  };
  if (a.K <= 8) pick_v(std::integral_constant<int, 8>{});
  else pick_v(std::integral_constant<int, 16>{});
  return hipGetLastError();
}

// ---- FP8 -> BF16 bridge: out = bf16(e4m3 * scale), sixteen codes per lane where a row allows it ---------------------------
template <bool kE8M0>
__device__ __forceinline__ float bridge_scale(const void* scales, int64_t at) {
  if constexpr (kE8M0) {
    const uint32_t b = static_cast<const uint8_t*>(scales)[at];
    return b ? bits_f32(b << 23) : bits_f32(0x00400000u);   // byte 0 is 2^-127; byte 255 reads as +inf here, as in the reference's bridge
  } else {
    return static_cast<const float*>(scales)[at];
  }
}
template <bool kE8M0>
__global__ __launch_bounds__(kFlatThreads) void fp8_bridge_kernel(const uint8_t* __restrict__ payload,
                                                                  const void* __restrict__ scales,
                                                                  uint16_t* __restrict__ out, int64_t rows, int64_t cols,
                                                                  int64_t scale_cols, int rs, int cs, int vec) {
  const int64_t units_per_row = (cols + 15) / 16;
  const int64_t u = static_cast<int64_t>(blockIdx.x) * kFlatThreads + threadIdx.x;
  if (u >= rows * units_per_row) return;
  const int64_t n = u / units_per_row, k0 = (u - n * units_per_row) * 16;
  const int64_t base = n * cols + k0;
  if (vec && k0 + 16 <= cols) {   // cs >= 4: the sixteen codes share one scale
    const float s = bridge_scale<kE8M0>(scales, (n >> rs) * scale_cols + (k0 >> cs));
    const uint4 p = *reinterpret_cast<const uint4*>(payload + base);
    const uint32_t w[4] = {p.x, p.y, p.z, p.w};
    uint32_t o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      o[2 * q + 0] = pack2_bf16(e4m3_to_f32(w[q] & 0xFFu) * s, e4m3_to_f32((w[q] >> 8) & 0xFFu) * s);
      o[2 * q + 1] = pack2_bf16(e4m3_to_f32((w[q] >> 16) & 0xFFu) * s, e4m3_to_f32(w[q] >> 24) * s);
    }
    uint4* dst = reinterpret_cast<uint4*>(out + base);
    dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
    dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
    return;
  }
  for (int64_t k = k0; k < cols && k < k0 + 16; ++k)
    out[n * cols + k] = f32_to_bf16(e4m3_to_f32(payload[n * cols + k]) * bridge_scale<kE8M0>(scales, (n >> rs) * scale_cols + (k >> cs)));
}

inline unsigned flat_blocks(int64_t lanes) { return static_cast<unsigned>((lanes + kFlatThreads - 1) / kFlatThreads); }

// ---- streaming probes (measurement harness) --------------------------------------------------------------------------------
// Plain copy, 16 bytes per lane per step, grid-stride: the calibration workload for a profiler's HBM byte counters.
__global__ __launch_bounds__(256) void probe_copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride)
    dst[i] = src[i];
}
// Plain read: a block owns a contiguous span and walks it with 16-byte loads, eight 4 KB lines in flight per block
// step (`span` != 0), or all lanes of the grid stride through the buffer together (`span` == 0); the loads are xor-ed
// together and one word per block is stored only if the result is a value no input produces — the rate a weight stream
// could reach with no arithmetic at all.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink,
                                                         int nontemporal, int span) {
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  const __attribute__((address_space(1))) u32x4_t* p = (const __attribute__((address_space(1))) u32x4_t*)(uintptr_t)src;
  constexpr int U = 8;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  size_t i, end, step;
  if (span) {
    const size_t per_block = (n16 + gridDim.x - 1) / gridDim.x;
    i = per_block * blockIdx.x + threadIdx.x;
    end = min(n16, per_block * (blockIdx.x + 1));
    step = blockDim.x;
  } else {
    i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    end = n16;
    step = static_cast<size_t>(gridDim.x) * blockDim.x;
  }
  for (; i + (U - 1) * step < end; i += U * step) {
    u32x4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = nontemporal ? __builtin_nontemporal_load(p + i + u * step) : p[i + u * step];
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  for (; i < end; i += step) acc ^= p[i];
  const uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (x == 0x9E3779B9u && sink != nullptr) sink[blockIdx.x] = x;
}

}  // namespace

hipError_t run_swiglu_clamp(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, float limit,
                            hipStream_t stream) {
  const int vec = ((reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  hipLaunchKernelGGL(swiglu_flat_kernel, dim3(flat_blocks((n + 7) / 8)), dim3(kFlatThreads), 0, stream, gate, up, out, n,
                     limit, vec);
  return hipGetLastError();
}

hipError_t run_gather_rows(const uint16_t* src, const int32_t* rows, uint16_t* dst, int n_rows, int hidden,
                           hipStream_t stream) {
  const bool vec = hidden % 8 == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
  const int unit = vec ? 8 : 1;
  const int per_row = hidden / unit;
  const int64_t units = static_cast<int64_t>(n_rows) * per_row;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(flat_blocks(units)), dim3(kFlatThreads), 0, stream, src, rows, dst, units,
                     per_row, unit, hidden);
  return hipGetLastError();
}

hipError_t run_accum(float* acc, const float* y, const int32_t* rows, const float* row_w, int n_rows, int hidden,
                     hipStream_t stream) {
  if (n_rows <= 0 || hidden <= 0) return hipSuccess;
  const bool vec = hidden % 4 == 0 && ((reinterpret_cast<uintptr_t>(acc) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
  const dim3 grid(static_cast<unsigned>(n_rows), static_cast<unsigned>((hidden + 4 * kFlatThreads - 1) / (4 * kFlatThreads)));
  if (vec)
    hipLaunchKernelGGL(scatter_fma_kernel<true>, grid, dim3(kFlatThreads), 0, stream, acc, y, rows, row_w, hidden);
  else
    hipLaunchKernelGGL(scatter_fma_kernel<false>, grid, dim3(kFlatThreads), 0, stream, acc, y, rows, row_w, hidden);
  return hipGetLastError();
}

hipError_t run_round_bf16(uint16_t* out, const float* acc, int64_t n, hipStream_t stream) {
  const int vec = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(acc)) & 15u) == 0;
  hipLaunchKernelGGL(round_flat_kernel, dim3(flat_blocks((n + 7) / 8)), dim3(kFlatThreads), 0, stream, out, acc, n, vec);
  return hipGetLastError();
}

hipError_t run_slot_accum(void* out, int out_f32, int with_shared, const float* contrib, const float* weights,
                          int tokens, int hidden, int top_k, hipStream_t stream) {
  ChainArgs a{};
  a.out = out;
  a.src = contrib;
  a.src_stride = static_cast<size_t>(hidden);
  a.weights = weights;
  a.shared = with_shared ? 1 : 0;
  a.K = top_k;
  a.hidden = hidden;
  return launch_chain<false>(a, out_f32, tokens, stream);
}

hipError_t run_accum_ordered(void* out, int out_f32, const void* down, int down_bf16, size_t down_stride,
                             const int32_t* slot_row, const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                             int top_k, int hidden, hipStream_t stream) {
  ChainArgs a{};
  a.out = out;
  a.src = static_cast<const float*>(down);
  a.src_bf16 = down_bf16;
  a.src_stride = down_stride;
  a.slot_row = slot_row;
  a.slot_ids = slot_ids;
  a.weights = slot_w;
  a.shared = shared_row0;
  a.K = top_k;
  a.hidden = hidden;
  return launch_chain<true>(a, out_f32, tokens, stream);
}

hipError_t run_fp8_dequant(const uint8_t* payload, const void* scales, int e8m0, uint16_t* out, int64_t rows,
                           int64_t cols, int rs, int cs, hipStream_t stream) {
  const int64_t scale_cols = (cols + (1LL << cs) - 1) >> cs;
  const int vec = cols % 16 == 0 && ((reinterpret_cast<uintptr_t>(payload) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const dim3 grid(flat_blocks(rows * ((cols + 15) / 16))), block(kFlatThreads);
  if (e8m0)
    hipLaunchKernelGGL(fp8_bridge_kernel<true>, grid, block, 0, stream, payload, scales, out, rows, cols, scale_cols, rs, cs, vec);
  else
    hipLaunchKernelGGL(fp8_bridge_kernel<false>, grid, block, 0, stream, payload, scales, out, rows, cols, scale_cols, rs, cs, vec);
  return hipGetLastError();
}

hipError_t run_probe_copy(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  const size_t n16 = bytes / 16;
  const size_t want = (n16 + 255) / 256;
  const unsigned blocks = static_cast<unsigned>(want < 1 ? 1 : (want > 16384 ? 16384 : want));
  hipLaunchKernelGGL(probe_copy_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<uint4*>(dst),
                     static_cast<const uint4*>(src), n16);
  return hipGetLastError();
}

hipError_t run_probe_read(const void* src, size_t bytes, void* sink, int nontemporal, int blocks, int span, hipStream_t stream) {
  const size_t n16 = bytes / 16;
  if (blocks <= 0) blocks = 2048;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(probe_read_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     static_cast<const uint4*>(src), n16, static_cast<uint32_t*>(sink), nontemporal, span);
  return hipGetLastError();
}

}  // namespace dgpp_amd
