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
// One wavefront per (expert, token): lanes stride the hidden vector in 16-byte vectors, each
// lane an fp32 fma chain in k order, then the butterfly.
constexpr int kRouterWaves = 4;

template <int kMode>
__global__ __launch_bounds__(kRouterWaves * kWaveSize) void router_dots_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ gate, const float* __restrict__ bias,
    float* __restrict__ scores, float* __restrict__ biased, int tokens, int hidden_dim, int n_experts,
    int vector_loads) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = blockIdx.x * kRouterWaves + wave;
  const int t = blockIdx.y;
  if (e >= n_experts || t >= tokens) return;
  const uint16_t* x = hidden + static_cast<size_t>(t) * hidden_dim;
  const uint16_t* w = gate + static_cast<size_t>(e) * hidden_dim;
  float dot = 0.f;
  if (vector_loads) {
    const int vecs = hidden_dim / 8;
    for (int v = lane; v < vecs; v += kWaveSize) {
      const uint4 xv = reinterpret_cast<const uint4*>(x)[v];
      const uint4 wv = reinterpret_cast<const uint4*>(w)[v];
      const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        dot = fmaf(bits_f32(xw[q] << 16), bits_f32(ww[q] << 16), dot);
        dot = fmaf(bits_f32(xw[q] & 0xFFFF0000u), bits_f32(ww[q] & 0xFFFF0000u), dot);
      }
    }
  } else {
    for (int k = lane; k < hidden_dim; k += kWaveSize) dot = fmaf(bf16_to_f32(x[k]), bf16_to_f32(w[k]), dot);
  }
  dot = wave_sum(dot);
  if (lane != 0) return;
  const size_t at = static_cast<size_t>(t) * n_experts + e;
  if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) {
    const float l = bf16_to_f32(f32_to_bf16(dot));
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

// The same dots for a batch of rows (sixteen and more): a wavefront keeps a TT x EE tile of (token, expert) sums, so a
// step's TT + EE vector loads feed TT * EE * 8 fmas and a gate row is fetched once per TT tokens instead of once per
// token. Every (token, expert) sum is still one wavefront's: lane l takes the 16-byte vectors l, l + 64, ... in
// ascending order, eight fmas each in element order, then the same butterfly - bit for bit the kernel above. Sixteen
// lanes then finish one score each. Counterpart of the reference's tiled dots (src/kernels/glm_moe.cu:735-835), which
// stages 16 x 16 tiles in shared memory; here the tile lives in registers and the L2 serves the re-reads.
constexpr int kTileExperts = 4;
constexpr int kRouterTiledFromTokens = 32;   // measured: below this the one-row form's many wavefronts win (the reference tiles from 16)

template <int kMode, int TT>
__global__ __launch_bounds__(kRouterWaves * kWaveSize) void router_dots_tile_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ gate, const float* __restrict__ bias,
    float* __restrict__ scores, float* __restrict__ biased, int tokens, int hidden_dim, int n_experts) {
  constexpr int EE = kTileExperts;
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
  const size_t at = static_cast<size_t>(t) * n_experts + e;
  if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) {
    const float l = bf16_to_f32(f32_to_bf16(mine));
    scores[at] = l;
    biased[at] = l;
  } else {
    float sc;
    if (kMode == DGPP_ROUTER_SQRT_SOFTPLUS_BIAS)
      sc = sqrtf(mine > 20.f ? mine : log1pf(expf(mine)));
    else
      sc = 1.0f / (1.0f + expf(-mine));
    scores[at] = sc;
    biased[at] = sc + bias[e];
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

hipError_t run_router_dots(int mode, const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                           float* biased, int tokens, int hidden_dim, int n_experts, hipStream_t stream, int allow_tiled) {
  const int vec = (hidden_dim % 8 == 0) && ((reinterpret_cast<uintptr_t>(hidden) & 15u) == 0) &&
                  ((reinterpret_cast<uintptr_t>(gate) & 15u) == 0);
  const int tuned = tune_get(kTuneRouterTile);   // bench / test switch: 2 or 4 forces the tiled form with that tile
  if (allow_tiled && vec && (tokens >= kRouterTiledFromTokens || tuned > 0)) {
    // Two tokens per wavefront (more wavefronts in flight) until the batch is large enough that four (fewer gate
    // re-reads) pays.
    const int tt = tuned > 0 ? (tuned >= 4 ? 4 : 2) : (tokens >= 128 ? 4 : 2);
    const dim3 grid((n_experts + kRouterWaves * kTileExperts - 1) / (kRouterWaves * kTileExperts), (tokens + tt - 1) / tt);
    const dim3 block(kRouterWaves * kWaveSize);
    auto go = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, block, 0, stream, hidden, gate, bias, scores, biased, tokens, hidden_dim, n_experts);
    };
    if (mode == DGPP_ROUTER_SOFTMAX_TOPK)
      tt == 4 ? go(router_dots_tile_kernel<DGPP_ROUTER_SOFTMAX_TOPK, 4>) : go(router_dots_tile_kernel<DGPP_ROUTER_SOFTMAX_TOPK, 2>);
    else if (mode == DGPP_ROUTER_SQRT_SOFTPLUS_BIAS)
      tt == 4 ? go(router_dots_tile_kernel<DGPP_ROUTER_SQRT_SOFTPLUS_BIAS, 4>)
              : go(router_dots_tile_kernel<DGPP_ROUTER_SQRT_SOFTPLUS_BIAS, 2>);
    else
      tt == 4 ? go(router_dots_tile_kernel<DGPP_ROUTER_SIGMOID_BIAS, 4>) : go(router_dots_tile_kernel<DGPP_ROUTER_SIGMOID_BIAS, 2>);
    return hipGetLastError();
  }
  const dim3 grid((n_experts + kRouterWaves - 1) / kRouterWaves, tokens);
  const dim3 block(kRouterWaves * kWaveSize);
  if (mode == DGPP_ROUTER_SOFTMAX_TOPK)
    hipLaunchKernelGGL(router_dots_kernel<DGPP_ROUTER_SOFTMAX_TOPK>, grid, block, 0, stream, hidden, gate, bias, scores,
                       biased, tokens, hidden_dim, n_experts, vec);
  else if (mode == DGPP_ROUTER_SQRT_SOFTPLUS_BIAS)
    hipLaunchKernelGGL(router_dots_kernel<DGPP_ROUTER_SQRT_SOFTPLUS_BIAS>, grid, block, 0, stream, hidden, gate, bias,
                       scores, biased, tokens, hidden_dim, n_experts, vec);
  else
    hipLaunchKernelGGL(router_dots_kernel<DGPP_ROUTER_SIGMOID_BIAS>, grid, block, 0, stream, hidden, gate, bias, scores,
                       biased, tokens, hidden_dim, n_experts, vec);
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
