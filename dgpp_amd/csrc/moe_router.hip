// The MoE router: score rows (one dot product per expert and token) and the top-k selection, alone or
// together with the decode slots' expert order.
//
// Reference counterparts in src/kernels/glm_moe.cu: router dots :86-196, selection :211-329, slot order :465-517.
// Ids given the scores are a bit-exact contract; the weights are fp32 chains in a defined order.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"
#include "gemv_core.hpp"
#include "moe_misc.hpp"
#include "moe_rank.hpp"
#include "numerics.hpp"
#include "router_select.hpp"

namespace dgpp_amd {
namespace {

using rsel::kWaveSize;
using rsel::select_token;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// ---- router ---------------------------------------------------------------------------------
// A finished dot becomes the token's score for the expert, and the score the selection ranks by
// (src/kernels/glm_moe.cu:86-196 defines the three modes).
template <int kMode>
__device__ __forceinline__ void store_score(float dot, const float* __restrict__ bias, int e, size_t at,
                                            float* __restrict__ scores, float* __restrict__ biased) {
  if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) {
    const float l = bf16_to_f32(f32_to_bf16(dot));   // the logit row is bf16-rounded
    scores[at] = l;
    biased[at] = l;
  } else {
    float sc;
    if (kMode == DGPP_ROUTER_SQRT_SOFTPLUS_BIAS)
      sc = sqrtf(dot > 20.f ? dot : log1pf(expf(dot)));
    else
      sc = 1.0f / (1.0f + expf(-dot));
    scores[at] = sc;
    biased[at] = sc + bias[e];
  }
}

// The score rows of a batch. A wavefront keeps a TT x EE tile of (token, expert) sums in registers: a step's TT + EE
// 16-byte vector loads feed TT * EE * 8 fmas, the next step's vectors are in flight while this step's fmas run, and a
// gate row is fetched once per TT tokens. Every (token, expert) sum is one wavefront's: lane l takes the vectors l,
// l + 64, ... in ascending order, eight fmas each in element order, then the butterfly - so the bits do not depend on
// the tile. TT = EE = 1 is the decode form (one wavefront per (token, expert): the most wavefronts in flight), larger
// tiles serve batches. The tile lives in registers and the L2 serves the re-reads, where the reference stages 16 x 16
// tiles in shared memory (src/kernels/glm_moe.cu:735-835).
constexpr int kRouterWaves = 4;
constexpr int kTileExperts = 4;
constexpr int kRouterTiledFromTokens = 32;   // measured: below this the one-row form's many wavefronts win (the reference tiles from 16)

template <int kMode, int TT, int EE>
__global__ __launch_bounds__(kRouterWaves * kWaveSize) void router_dots_tile_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ gate, const float* __restrict__ bias,
    float* __restrict__ scores, float* __restrict__ biased, int tokens, int hidden_dim, int n_experts) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e0 = (blockIdx.x * kRouterWaves + wave) * EE;
  const int t0 = blockIdx.y * TT;
  if (e0 >= n_experts) return;
  const uint4* x[TT];
  const uint4* w[EE];
#pragma unroll
  for (int i = 0; i < TT; ++i)   // rows past the batch repeat its last row; their sums are never stored
    x[i] = reinterpret_cast<const uint4*>(hidden + static_cast<size_t>(min(t0 + i, tokens - 1)) * hidden_dim);
#pragma unroll
  for (int j = 0; j < EE; ++j)
    w[j] = reinterpret_cast<const uint4*>(gate + static_cast<size_t>(min(e0 + j, n_experts - 1)) * hidden_dim);
  float dot[TT][EE];
#pragma unroll
  for (int i = 0; i < TT; ++i)
#pragma unroll
    for (int j = 0; j < EE; ++j) dot[i][j] = 0.f;
  const int vecs = hidden_dim / 8;
  uint4 xn[TT], wn[EE];   // the next step's vectors, in flight while this step's fmas run
  auto fetch = [&](int v) {
    const int at = v < vecs ? v : lane;   // past the end: a harmless re-read, never used
#pragma unroll
    for (int i = 0; i < TT; ++i) xn[i] = x[i][at];
#pragma unroll
    for (int j = 0; j < EE; ++j) wn[j] = w[j][at];
  };
  if (lane < vecs) fetch(lane);
  for (int v = lane; v < vecs; v += kWaveSize) {
    uint4 xv[TT], wv[EE];
#pragma unroll
    for (int i = 0; i < TT; ++i) xv[i] = xn[i];
#pragma unroll
    for (int j = 0; j < EE; ++j) wv[j] = wn[j];
    fetch(v + kWaveSize);
#pragma unroll
    for (int i = 0; i < TT; ++i) {
      const uint32_t xw[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
#pragma unroll
      for (int j = 0; j < EE; ++j) {
        const uint32_t ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
        float d = dot[i][j];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          d = fmaf(bits_f32(xw[q] << 16), bits_f32(ww[q] << 16), d);
          d = fmaf(bits_f32(xw[q] & 0xFFFF0000u), bits_f32(ww[q] & 0xFFFF0000u), d);
        }
        dot[i][j] = d;
      }
    }
  }
  float mine = 0.f;   // lane i * EE + j finishes the tile's (i, j) score
#pragma unroll
  for (int i = 0; i < TT; ++i)
#pragma unroll
    for (int j = 0; j < EE; ++j) {
      const float s = wave_sum(dot[i][j]);
      if (lane == i * EE + j) mine = s;
    }
  const int t = t0 + lane / EE, e = e0 + lane % EE;
  if (lane >= TT * EE || t >= tokens || e >= n_experts) return;
  store_score<kMode>(mine, bias, e, static_cast<size_t>(t) * n_experts + e, scores, biased);
}

// Rows that cannot be read as aligned 16-byte vectors (hidden not a multiple of eight, unaligned pointers): a
// wavefront per (token, expert), lanes a stride of 64 elements apart.
template <int kMode>
__global__ __launch_bounds__(kRouterWaves * kWaveSize) void router_dots_unaligned_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ gate, const float* __restrict__ bias,
    float* __restrict__ scores, float* __restrict__ biased, int tokens, int hidden_dim, int n_experts) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * kRouterWaves + (threadIdx.x >> 6), t = blockIdx.y;
  if (e >= n_experts || t >= tokens) return;
  const uint16_t* x = hidden + static_cast<size_t>(t) * hidden_dim;
  const uint16_t* w = gate + static_cast<size_t>(e) * hidden_dim;
  float dot = 0.f;
  for (int k = lane; k < hidden_dim; k += kWaveSize) dot = fmaf(bf16_to_f32(x[k]), bf16_to_f32(w[k]), dot);
  dot = wave_sum(dot);
  if (lane == 0) store_score<kMode>(dot, bias, e, static_cast<size_t>(t) * n_experts + e, scores, biased);
}

// ---- the MiniMax router (src/kernels/minimax.hpp:56-60, src/kernels/minimax.cu:397-440) ---------------------------
// FP32 gate rows against BF16 token rows; the score is the sigmoid of the FP32 dot and is what the weights are made
// of, the bias enters the ranking only. One wavefront per (row, expert): lane l takes the eight-element groups l,
// l + 64, ... in ascending order (one 16-byte load of the token row, two of the gate row), eight fmas each in element
// order, then the butterfly; rows that are not 32-byte aligned groups go element by element.
__global__ __launch_bounds__(kRouterWaves * kWaveSize) void minimax_router_dots_kernel(
    const uint16_t* __restrict__ x, const float* __restrict__ gate, float* __restrict__ scores, int rows, int hidden,
    int experts, int vectors) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * kRouterWaves + (threadIdx.x >> 6), r = blockIdx.y;
  if (e >= experts || r >= rows) return;
  const uint16_t* xr = x + static_cast<size_t>(r) * hidden;
  const float* w = gate + static_cast<size_t>(e) * hidden;
  float dot = 0.f;
  if (vectors) {
    for (int v = lane; v < hidden / 8; v += kWaveSize) {
      const uint4 xv = reinterpret_cast<const uint4*>(xr)[v];
      const float4 w0 = reinterpret_cast<const float4*>(w)[2 * v], w1 = reinterpret_cast<const float4*>(w)[2 * v + 1];
      dot = fmaf(bits_f32(xv.x << 16), w0.x, dot);
      dot = fmaf(bits_f32(xv.x & 0xFFFF0000u), w0.y, dot);
      dot = fmaf(bits_f32(xv.y << 16), w0.z, dot);
      dot = fmaf(bits_f32(xv.y & 0xFFFF0000u), w0.w, dot);
      dot = fmaf(bits_f32(xv.z << 16), w1.x, dot);
      dot = fmaf(bits_f32(xv.z & 0xFFFF0000u), w1.y, dot);
      dot = fmaf(bits_f32(xv.w << 16), w1.z, dot);
      dot = fmaf(bits_f32(xv.w & 0xFFFF0000u), w1.w, dot);
    }
  } else {
    for (int k = lane; k < hidden; k += kWaveSize) dot = fmaf(bf16_to_f32(xr[k]), w[k], dot);
  }
  dot = wave_sum(dot);
  if (lane == 0) scores[static_cast<size_t>(r) * experts + e] = 1.0f / (1.0f + expf(-dot));
}
template <int PER_LANE>
__global__ __launch_bounds__(kWaveSize) void minimax_router_select_kernel(const float* __restrict__ scores,
                                                                          const float* __restrict__ bias,
                                                                          int32_t* __restrict__ ids, float* __restrict__ weights,
                                                                          int rows, int experts, int top_k, float factor) {
  const int r = blockIdx.x, lane = threadIdx.x;
  if (r >= rows) return;
  int id;
  float w;
  select_token<DGPP_ROUTER_SIGMOID_BIAS, PER_LANE, true>(scores + static_cast<size_t>(r) * experts, bias, experts, top_k, factor, 1,
                                                         lane, id, w);
  if (lane < top_k) {
    ids[static_cast<size_t>(r) * top_k + lane] = id;
    weights[static_cast<size_t>(r) * top_k + lane] = w;
  }
}

// One wavefront per token, the whole score row in registers (router_select.hpp): 64 * PER_LANE experts.
template <int kMode, int PER_LANE>
__global__ __launch_bounds__(kWaveSize) void router_select_reg_kernel(
    const float* __restrict__ scores, const float* __restrict__ biased, int32_t* __restrict__ ids,
    float* __restrict__ weights, int tokens, int n_experts, int top_k, float scaling, int norm_topk) {
  const int t = blockIdx.x, lane = threadIdx.x;
  if (t >= tokens) return;
  const size_t row = static_cast<size_t>(t) * n_experts;
  int id;
  float w;
  select_token<kMode, PER_LANE>(scores + row, biased + row, n_experts, top_k, scaling, norm_topk, lane, id, w);
  if (lane < top_k) {
    ids[static_cast<size_t>(t) * top_k + lane] = id;
    weights[static_cast<size_t>(t) * top_k + lane] = w;
  }
}

// Selection and slot order in ONE launch for a decode batch: one wavefront per token selects, the
// block then ranks the slots by (expert, slot) exactly as slot_order_kernel does (key = expert id,
// or n_experts for the token's shared slot). tokens * 64 threads, tokens <= 16.
template <int kMode, int PER_LANE>
__global__ __launch_bounds__(1024) void router_select_order_kernel(
    const float* __restrict__ scores, const float* __restrict__ biased, int32_t* __restrict__ ids,
    float* __restrict__ weights, int32_t* __restrict__ order, int tokens, int n_experts, int top_k, float scaling,
    int norm_topk, int shared_early) {
  __shared__ __align__(16) int32_t keys[16 * 17 + 4];
  const int t = threadIdx.x >> 6, lane = threadIdx.x & (kWaveSize - 1);
  const size_t row = static_cast<size_t>(t) * n_experts;
  int id;
  float w;
  select_token<kMode, PER_LANE>(scores + row, biased + row, n_experts, top_k, scaling, norm_topk, lane, id, w);
  if (lane < top_k) {
    ids[static_cast<size_t>(t) * top_k + lane] = id;
    weights[static_cast<size_t>(t) * top_k + lane] = w;
    keys[t * (top_k + 1) + lane] = slot_sort_key(id, t * (top_k + 1) + lane);
  } else if (lane == top_k) {
    keys[t * (top_k + 1) + lane] = slot_sort_key(n_experts, t * (top_k + 1) + lane);
  }
  if (order == nullptr) return;
  const int slots = tokens * (top_k + 1);
  const int padded = (slots + 3) & ~3;
  if (threadIdx.x < padded - slots) keys[slots + threadIdx.x] = INT_MAX;
  __syncthreads();
  const int s = threadIdx.x;
  if (s >= slots) return;
  int pos = slot_rank(keys, padded, keys[s]);
  if (shared_early) {
    const int routed = tokens * top_k;
    pos = pos < routed ? pos + (pos < tokens ? pos : tokens) : 2 * (pos - routed) + 1;
  }
  order[pos] = s;
}

// Routes taken from a table instead of the scores' top k (src/kernels/glm_moe.cu:917-949): token t's experts are row
// tokens[t] of tid2eid (ascending ids), its weights the scores at those ids, normalised and scaled as the selection
// does: the sum runs over the row in order from zero, + 1e-20, one division per weight. One lane per (token, slot);
// every lane of a token walks the row's sum itself (top_k <= 16 scores out of one or two cache lines), so the routes
// leave as coalesced stores.
__global__ __launch_bounds__(256) void hash_routes_kernel(const int64_t* __restrict__ tokens, const int32_t* __restrict__ tid2eid,
                                                          const float* __restrict__ scores, int32_t* __restrict__ ids,
                                                          float* __restrict__ weights, int n_tokens, int vocab, int n_experts,
                                                          int top_k, float scaling, int norm_topk) {
  const int64_t at = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (at >= static_cast<int64_t>(n_tokens) * top_k) return;
  const int t = static_cast<int>(at / top_k), i = static_cast<int>(at - static_cast<int64_t>(t) * top_k);
  int64_t tok = tokens[t];
  if (tok < 0 || tok >= vocab) tok = 0;   // a padding row: any table row (its output is never read)
  const int32_t* row = tid2eid + tok * top_k;
  const float* sc = scores + static_cast<size_t>(t) * n_experts;
  float denom = 0.f, mine = 0.f;
  for (int j = 0; j < top_k; ++j) {
    const float v = sc[row[j]];
    denom = denom + v;
    if (j == i) mine = v;
  }
  denom = denom + 1e-20f;
  ids[at] = row[i];
  weights[at] = norm_topk ? (mine / denom) * scaling : mine * scaling;
}

}  // namespace

hipError_t run_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int32_t* ids, float* weights,
                           int n_tokens, int vocab, int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream) {
  const int64_t lanes = static_cast<int64_t>(n_tokens) * top_k;
  hipLaunchKernelGGL(hash_routes_kernel, dim3(static_cast<unsigned>((lanes + 255) / 256)), dim3(256), 0, stream, tokens, tid2eid,
                     scores, ids, weights, n_tokens, vocab, n_experts, top_k, scaling, norm_topk);
  return hipGetLastError();
}

template <int TT, int EE>
static void launch_dots_tile(int mode, dim3 grid, hipStream_t stream, const uint16_t* hidden, const uint16_t* gate,
                             const float* bias, float* scores, float* biased, int tokens, int hidden_dim, int n_experts) {
  const dim3 block(kRouterWaves * kWaveSize);
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, grid, block, 0, stream, hidden, gate, bias, scores, biased, tokens, hidden_dim, n_experts);
  };
  if (mode == DGPP_ROUTER_SOFTMAX_TOPK) go(router_dots_tile_kernel<DGPP_ROUTER_SOFTMAX_TOPK, TT, EE>);
  else if (mode == DGPP_ROUTER_SQRT_SOFTPLUS_BIAS) go(router_dots_tile_kernel<DGPP_ROUTER_SQRT_SOFTPLUS_BIAS, TT, EE>);
  else go(router_dots_tile_kernel<DGPP_ROUTER_SIGMOID_BIAS, TT, EE>);
}

hipError_t run_router_dots(int mode, const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                           float* biased, int tokens, int hidden_dim, int n_experts, hipStream_t stream, int allow_tiled) {
  const bool vec = (hidden_dim % 8 == 0) && ((reinterpret_cast<uintptr_t>(hidden) & 15u) == 0) &&
                   ((reinterpret_cast<uintptr_t>(gate) & 15u) == 0);
  if (!vec) {
    const dim3 grid((n_experts + kRouterWaves - 1) / kRouterWaves, tokens), block(kRouterWaves * kWaveSize);
    auto go = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, block, 0, stream, hidden, gate, bias, scores, biased, tokens, hidden_dim, n_experts);
    };
    if (mode == DGPP_ROUTER_SOFTMAX_TOPK) go(router_dots_unaligned_kernel<DGPP_ROUTER_SOFTMAX_TOPK>);
    else if (mode == DGPP_ROUTER_SQRT_SOFTPLUS_BIAS) go(router_dots_unaligned_kernel<DGPP_ROUTER_SQRT_SOFTPLUS_BIAS>);
    else go(router_dots_unaligned_kernel<DGPP_ROUTER_SIGMOID_BIAS>);
    return hipGetLastError();
  }
  const int tuned = tune_get(kTuneRouterTile);   // bench / test switch: 2 or 4 forces the tiled form with that tile
  if (allow_tiled && (tokens >= kRouterTiledFromTokens || tuned > 0)) {
    // Two tokens per wavefront (more wavefronts in flight) until the batch is large enough that four (fewer gate
    // re-reads) pays.
    const int tt = tuned > 0 ? (tuned >= 4 ? 4 : 2) : (tokens >= 128 ? 4 : 2);
    const dim3 grid((n_experts + kRouterWaves * kTileExperts - 1) / (kRouterWaves * kTileExperts), (tokens + tt - 1) / tt);
    if (tt == 4) launch_dots_tile<4, kTileExperts>(mode, grid, stream, hidden, gate, bias, scores, biased, tokens, hidden_dim, n_experts);
    else launch_dots_tile<2, kTileExperts>(mode, grid, stream, hidden, gate, bias, scores, biased, tokens, hidden_dim, n_experts);
    return hipGetLastError();
  }
  const dim3 grid((n_experts + kRouterWaves - 1) / kRouterWaves, tokens);
  launch_dots_tile<1, 1>(mode, grid, stream, hidden, gate, bias, scores, biased, tokens, hidden_dim, n_experts);
  return hipGetLastError();
}

// PER_LANE for a row of n_experts (<= 4096, the configuration's limit): the smallest power of two that holds it.
template <int kMode, int PER_LANE>
static void launch_select_reg(const float* scores, const float* biased, int32_t* ids, float* weights, int tokens,
                              int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream) {
  hipLaunchKernelGGL((router_select_reg_kernel<kMode, PER_LANE>), dim3(tokens), dim3(kWaveSize), 0, stream, scores, biased,
                     ids, weights, tokens, n_experts, top_k, scaling, norm_topk);
}
template <int kMode>
static void launch_select_mode(const float* scores, const float* biased, int32_t* ids, float* weights, int tokens,
                               int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream) {
  const int per_lane = (n_experts + kWaveSize - 1) / kWaveSize;
  if (per_lane <= 4) launch_select_reg<kMode, 4>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
  else if (per_lane <= 8) launch_select_reg<kMode, 8>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
  else if (per_lane <= 16) launch_select_reg<kMode, 16>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
  else if (per_lane <= 32) launch_select_reg<kMode, 32>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
  else launch_select_reg<kMode, 64>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
}

hipError_t run_router_select(int mode, const float* scores, const float* biased, int32_t* ids, float* weights,
                             int tokens, int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream) {
  if (n_experts > 64 * kWaveSize) return hipErrorInvalidValue;   // the configuration check stops at 4096 experts
  if (mode == DGPP_ROUTER_SOFTMAX_TOPK)
    launch_select_mode<DGPP_ROUTER_SOFTMAX_TOPK>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
  else
    launch_select_mode<DGPP_ROUTER_SIGMOID_BIAS>(scores, biased, ids, weights, tokens, n_experts, top_k, scaling, norm_topk, stream);
  return hipGetLastError();
}

hipError_t run_minimax_router(const uint16_t* x, const float* gate, const float* bias, int rows, int hidden, int experts,
                              int top_k, float factor, float* scores, int32_t* ids, float* weights, hipStream_t stream) {
  if (experts > 64 * kWaveSize) return hipErrorInvalidValue;
  const int vectors = hidden % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(gate) & 15u) == 0;
  hipLaunchKernelGGL(minimax_router_dots_kernel, dim3((experts + kRouterWaves - 1) / kRouterWaves, rows),
                     dim3(kRouterWaves * kWaveSize), 0, stream, x, gate, scores, rows, hidden, experts, vectors);
  const int per_lane = (experts + kWaveSize - 1) / kWaveSize;
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(rows), dim3(kWaveSize), 0, stream, scores, bias, ids, weights, rows, experts, top_k, factor);
  };
  if (per_lane <= 4) go(minimax_router_select_kernel<4>);
  else if (per_lane <= 8) go(minimax_router_select_kernel<8>);
  else if (per_lane <= 16) go(minimax_router_select_kernel<16>);
  else if (per_lane <= 32) go(minimax_router_select_kernel<32>);
  else go(minimax_router_select_kernel<64>);
  return hipGetLastError();
}

hipError_t run_router_select_order(int mode, const float* scores, const float* biased, int32_t* ids, float* weights,
                                   int32_t* order, int tokens, int n_experts, int top_k, float scaling, int norm_topk,
                                   int shared_early, hipStream_t stream) {
  const bool softmax = mode == DGPP_ROUTER_SOFTMAX_TOPK;
  const dim3 grid(1), block(tokens * kWaveSize);
  if (n_experts <= 4 * kWaveSize) {
    if (softmax)
      hipLaunchKernelGGL((router_select_order_kernel<DGPP_ROUTER_SOFTMAX_TOPK, 4>), grid, block, 0, stream, scores,
                         biased, ids, weights, order, tokens, n_experts, top_k, scaling, norm_topk, shared_early);
    else
      hipLaunchKernelGGL((router_select_order_kernel<DGPP_ROUTER_SIGMOID_BIAS, 4>), grid, block, 0, stream, scores,
                         biased, ids, weights, order, tokens, n_experts, top_k, scaling, norm_topk, shared_early);
  } else {
    if (softmax)
      hipLaunchKernelGGL((router_select_order_kernel<DGPP_ROUTER_SOFTMAX_TOPK, 8>), grid, block, 0, stream, scores,
                         biased, ids, weights, order, tokens, n_experts, top_k, scaling, norm_topk, shared_early);
    else
      hipLaunchKernelGGL((router_select_order_kernel<DGPP_ROUTER_SIGMOID_BIAS, 8>), grid, block, 0, stream, scores,
                         biased, ids, weights, order, tokens, n_experts, top_k, scaling, norm_topk, shared_early);
  }
  return hipGetLastError();
}

}  // namespace dgpp_amd
