// Router, token->expert grouping, and the elementwise / accumulation kernels of the MoE path.
// Integer outputs (ids given scores, rows, slot_row, segments, order, tiles) are bit-exact
// contracts; the fp32 accumulation chains are fmaf sequences in a defined order.
//
// Reference counterparts in src/kernels/glm_moe.cu: router :86-329, swiglu :331-347, gather
// :349-359, accum / round :371-393, slot order :465-517, slot accum :673-711, segmentation
// :1382-1439, ordered accumulation :1446-1489, tile list :1553-1569; src/kernels/minimax.cu:33-50
// (segment compaction); src/kernels/fp8_dequant.cu:33-50.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"
#include "moe_misc.hpp"
#include "numerics.hpp"
#include "router_select.hpp"

namespace dgpp_amd {
namespace {

constexpr int kElemThreads = 256;
using rsel::kWaveSize;
using rsel::select_token;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// Exclusive prefix sum of one int per thread over a block of up to 1024 threads; *total gets
// the block sum. s_wave needs 16 ints. Ends with a barrier, so s_wave may be reused at once.
__device__ __forceinline__ int block_exclusive_scan(int v, int* s_wave, int* total) {
  const int lane = threadIdx.x & (kWaveSize - 1), wave = threadIdx.x >> 6;
  const int n_waves = (blockDim.x + kWaveSize - 1) >> 6;
  int x = v;
#pragma unroll
  for (int off = 1; off < kWaveSize; off <<= 1) {
    const int y = __shfl_up(x, off);
    if (lane >= off) x += y;
  }
  if (lane == kWaveSize - 1) s_wave[wave] = x;
  __syncthreads();
  int base = 0, sum = 0;
  for (int w = 0; w < n_waves; ++w) {
    const int c = s_wave[w];
    if (w < wave) base += c;
    sum += c;
  }
  *total = sum;
  __syncthreads();
  return base + x - v;
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

// One wavefront per token: top-k over the biased row with strict '>' (the lower id wins a tie),
// ids sorted ascending, weights w / (sum + 1e-20) * scale with a true division per element;
// softmax mode turns the logit row into fp32 probabilities first and rounds the weights to bf16.
template <int kMode>
__global__ __launch_bounds__(kWaveSize) void router_select_kernel(
    const float* __restrict__ scores, const float* __restrict__ biased, int32_t* __restrict__ ids,
    float* __restrict__ weights, int tokens, int n_experts, int top_k, float scaling, int norm_topk) {
  extern __shared__ float sel_lds[];  // [2][n_experts]
  float* s_scores = sel_lds;
  float* s_biased = sel_lds + n_experts;
  const int t = blockIdx.x, lane = threadIdx.x;
  if (t >= tokens) return;
  const size_t row = static_cast<size_t>(t) * n_experts;
  for (int e = lane; e < n_experts; e += kWaveSize) {
    s_scores[e] = scores[row + e];
    s_biased[e] = biased[row + e];
  }
  __syncthreads();
  if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) {
    float m = -INFINITY;
    for (int e = lane; e < n_experts; e += kWaveSize) m = fmaxf(m, s_scores[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < n_experts; e += kWaveSize) sum += expf(s_scores[e] - m);
    sum = wave_sum(sum);
    for (int e = lane; e < n_experts; e += kWaveSize) s_scores[e] = expf(s_scores[e] - m) / sum;
    __syncthreads();
  }
  int sel[16];
  float wsel[16];
  for (int r = 0; r < top_k; ++r) {
    int best = INT_MAX;
    float bv = -INFINITY;
    for (int e = lane; e < n_experts; e += kWaveSize) {
      const float v = s_biased[e];
      if (v > bv) {
        bv = v;
        best = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off);
      const int oid = __shfl_xor(best, off);
      if (ov > bv || (ov == bv && oid < best)) {
        bv = ov;
        best = oid;
      }
    }
    if (best == INT_MAX) best = 0;  // a row of -inf / NaN keys: stay in bounds
    sel[r] = best;
    wsel[r] = s_scores[best];
    __syncthreads();
    if (lane == 0) s_biased[best] = -INFINITY;
    __syncthreads();
  }
  if (lane != 0) return;
  for (int i = 1; i < top_k; ++i) {  // ascending expert id
    const int id = sel[i];
    const float w = wsel[i];
    int j = i - 1;
    while (j >= 0 && sel[j] > id) {
      sel[j + 1] = sel[j];
      wsel[j + 1] = wsel[j];
      --j;
    }
    sel[j + 1] = id;
    wsel[j + 1] = w;
  }
  float denom = 0.f;
  for (int i = 0; i < top_k; ++i) denom += wsel[i];
  denom += 1e-20f;
  for (int i = 0; i < top_k; ++i) {
    float w = norm_topk ? (wsel[i] / denom) * scaling : wsel[i] * scaling;
    if (kMode == DGPP_ROUTER_SOFTMAX_TOPK) w = bf16_to_f32(f32_to_bf16(w));
    ids[static_cast<size_t>(t) * top_k + i] = sel[i];
    weights[static_cast<size_t>(t) * top_k + i] = w;
  }
}

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

// Ranks by (key, slot) as one integer: key << 10 | slot (slots < 1024, keys <= n_experts < 2^16), unique per slot.
__device__ __forceinline__ int32_t slot_sort_key(int key, int slot) { return (key << 10) | slot; }
// Rank of a slot among `padded` such integers (a multiple of 4; pad entries hold INT_MAX): how many are below
// `mine`. Four per LDS read, one compare and one add each: the ranking is bound by the vector ALU.
__device__ __forceinline__ int slot_rank(const int32_t* __restrict__ sort_keys, int padded, int32_t mine) {
  const int4* k4 = reinterpret_cast<const int4*>(sort_keys);
  int pos = 0;
#pragma unroll 4
  for (int o = 0; o < padded / 4; ++o) {
    const int4 v = k4[o];
    pos += (v.x < mine) + (v.y < mine) + (v.z < mine) + (v.w < mine);
  }
  return pos;
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

// ---- elementwise ------------------------------------------------------------------------------
__global__ void swiglu_clamp_kernel(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up,
                                    uint16_t* __restrict__ out, int64_t n, float limit) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float g = bf16_to_f32(gate[i]);
  float u = bf16_to_f32(up[i]);
  if (g > limit) g = limit;
  u = fminf(fmaxf(u, -limit), limit);
  const uint16_t t = f32_to_bf16(g * (1.0f / (1.0f + expf(-g))));
  out[i] = f32_to_bf16(bf16_to_f32(t) * u);
}

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

__global__ void accum_kernel(float* __restrict__ acc, const float* __restrict__ y, const int32_t* __restrict__ rows,
                             const float* __restrict__ row_w, int64_t n, int hidden) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t r = i / hidden;
  float* dst = acc + static_cast<int64_t>(rows[r]) * hidden + (i - r * hidden);
  *dst = fmaf(row_w[r], y[i], *dst);
}

__global__ void round_bf16_kernel(uint16_t* __restrict__ out, const float* __restrict__ acc, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  out[i] = f32_to_bf16(acc[i]);
}

// Slot-layout chain: a = 0; a = fma(w_j, y_j, a) for j ascending; then the shared row with
// weight 1; one rounding (or none).
template <bool kShared, bool kF32>
__global__ void slot_accum_kernel(void* __restrict__ out, const float* __restrict__ contrib,
                                  const float* __restrict__ weights, int64_t n, int hidden, int top_k) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / hidden;
  const int c = static_cast<int>(i - t * hidden);
  const int64_t base = t * (top_k + 1);
  float a = 0.f;
  for (int j = 0; j < top_k; ++j)
    a = fmaf(weights[t * top_k + j], contrib[(base + j) * hidden + c], a);
  if (kShared) a = fmaf(1.0f, contrib[(base + top_k) * hidden + c], a);
  if (kF32)
    static_cast<float*>(out)[i] = a;
  else
    static_cast<uint16_t*>(out)[i] = f32_to_bf16(a);
}

// Grouped-layout chain: the token's slots visited in ascending expert id (stable), rows found
// through slot_row, then the shared row at shared_row0 + t when shared_row0 >= 0.
template <bool kF32>
__global__ void accum_ordered_kernel(void* __restrict__ out, const float* __restrict__ down, size_t down_stride,
                                     const int32_t* __restrict__ slot_row, const int32_t* __restrict__ slot_ids,
                                     const float* __restrict__ slot_w, int shared_row0, int tokens, int K,
                                     int hidden) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<int64_t>(tokens) * hidden) return;
  const int t = static_cast<int>(i / hidden);
  const int h = static_cast<int>(i - static_cast<int64_t>(t) * hidden);
  int ord[16];
  for (int j = 0; j < K; ++j) ord[j] = j;
  for (int j = 1; j < K; ++j) {
    const int cur = ord[j], key = slot_ids[t * K + cur];
    int p = j - 1;
    while (p >= 0 && slot_ids[t * K + ord[p]] > key) {
      ord[p + 1] = ord[p];
      --p;
    }
    ord[p + 1] = cur;
  }
  float acc = 0.f;
  for (int j = 0; j < K; ++j) {
    const int s = t * K + ord[j];
    acc = fmaf(slot_w[s], down[static_cast<size_t>(slot_row[s]) * down_stride + h], acc);
  }
  if (shared_row0 >= 0) acc = fmaf(1.0f, down[static_cast<size_t>(shared_row0 + t) * down_stride + h], acc);
  if (kF32)
    static_cast<float*>(out)[i] = acc;
  else
    static_cast<uint16_t*>(out)[i] = f32_to_bf16(acc);
}

// ---- grouping ------------------------------------------------------------------------------------
// One block per expert plus one for the shared segment, ONE launch: a block derives its own
// segment start as the number of ids below its expert (no cross-block dependency), then places
// its (token, slot) pairs in (token, slot) order with a block scan over match flags — the host
// path's stable counting sort, src/models/glm/moe_layer.cpp:634-659.
constexpr int kSegThreads = 256;
__global__ __launch_bounds__(kSegThreads) void segment_kernel(const int32_t* __restrict__ ids, int tokens, int K,
                                                              int E, int32_t* __restrict__ rows,
                                                              int32_t* __restrict__ slot_row,
                                                              DgppMoeSegment* __restrict__ segs) {
  __shared__ int s_wave[16];
  __shared__ int s_less, s_equal;
  const int e = blockIdx.x;
  const int tk = tokens * K;
  if (e == E) {  // the shared expert: every token once more, after the routed rows
    for (int t = threadIdx.x; t < tokens; t += kSegThreads) rows[tk + t] = t;
    if (threadIdx.x == 0) segs[E] = DgppMoeSegment{tk, tokens, E};
    return;
  }
  if (threadIdx.x == 0) {
    s_less = 0;
    s_equal = 0;
  }
  __syncthreads();
  int less = 0, equal = 0;
  for (int i = threadIdx.x; i < tk; i += kSegThreads) {
    const int id = ids[i];
    less += id < e;
    equal += id == e;
  }
  // Integer sums: the order of the atomic adds does not change the result.
  if (less) atomicAdd(&s_less, less);
  if (equal) atomicAdd(&s_equal, equal);
  __syncthreads();
  const int row0 = s_less, count = s_equal;
  if (threadIdx.x == 0) segs[e] = DgppMoeSegment{row0, count, e};
  if (count == 0) return;
  int running = row0;
  for (int base = 0; base < tk; base += kSegThreads) {
    const int i = base + threadIdx.x;
    const int flag = (i < tk && ids[i] == e) ? 1 : 0;
    int total = 0;
    const int excl = block_exclusive_scan(flag, s_wave, &total);
    if (flag) {
      const int pos = running + excl;
      rows[pos] = i / K;
      slot_row[i] = pos;
    }
    running += total;
  }
}

// One block, one thread per slot: rank by (key, slot), key = expert id or E for the shared slot.
__global__ void slot_order_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ order,
                                  int32_t* __restrict__ runs, int slots, int top_k, int n_experts,
                                  int shared_early) {
  extern __shared__ __align__(16) int32_t so_lds[];  // keys [slots padded to 4]; with runs: sorted [slots], groups [slots]
  const int padded = (slots + 3) & ~3;
  int32_t* keys = so_lds;
  int32_t* sorted = keys + padded;
  int32_t* groups = sorted + slots;
  const int s = threadIdx.x;
  if (s < slots) {
    const int t = s / (top_k + 1), j = s - t * (top_k + 1);
    keys[s] = slot_sort_key(j < top_k ? ids[static_cast<size_t>(t) * top_k + j] : n_experts, s);
  } else if (s < padded) {
    keys[s] = INT_MAX;
  }
  __syncthreads();
  if (s < slots) {
    const int mine = keys[s] >> 10;
    int pos = slot_rank(keys, padded, keys[s]);
    if (shared_early) {
      const int tokens = slots / (top_k + 1), routed = tokens * top_k;
      pos = pos < routed ? pos + (pos < tokens ? pos : tokens) : 2 * (pos - routed) + 1;
    }
    order[pos] = s;
    if (runs) sorted[pos] = mine;
  }
  if (!runs) return;
  __syncthreads();
  constexpr int kTileRows = 16, kGroupRows = 64;
  int len = 0;
  if (s < slots) {
    if (s == 0 || sorted[s - 1] != sorted[s]) {
      len = 1;
      while (s + len < slots && sorted[s + len] == sorted[s]) ++len;
    }
    runs[s] = len;
    groups[s] = len > kTileRows ? (len + kGroupRows - 1) / kGroupRows : 0;
  }
  __syncthreads();
  if (s < slots) {
    int base = 0;
    for (int o = 0; o < s; ++o) base += groups[o];
    int32_t* list = runs + slots;
    for (int g = 0; g < groups[s]; ++g) {
      const int r0 = g * kGroupRows;
      list[base + g] = (s + r0) | (min(kGroupRows, len - r0) << 16);
    }
    if (s == slots - 1)
      for (int i = base + groups[s]; i < slots / (kTileRows + 1) + 1; ++i) list[i] = -1;
  }
}

// The same order from several blocks (no run list): every block builds all sort keys in its LDS and ranks its own
// 32 slots with four lanes each, so the ranking's vector work spreads over CUs instead of queueing on one.
constexpr int kOrderThreads = 128;
__global__ __launch_bounds__(kOrderThreads) void slot_order_wide_kernel(const int32_t* __restrict__ ids,
                                                                        int32_t* __restrict__ order, int slots, int top_k,
                                                                        int n_experts, int shared_early) {
  extern __shared__ __align__(16) int32_t sw_lds[];   // sort keys [slots padded to 4]
  const int padded = (slots + 3) & ~3;
  // at most 1024 slots: eight per thread, every id load issued before the first is used
  int32_t v[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int i = threadIdx.x + u * kOrderThreads;
    const int c = i < slots ? i : 0;
    const int t = c / (top_k + 1), j = c - t * (top_k + 1);
    v[u] = ids[static_cast<size_t>(t) * top_k + (j < top_k ? j : 0)];
    v[u] = i < slots ? slot_sort_key(j < top_k ? v[u] : n_experts, i) : INT_MAX;
  }
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int i = threadIdx.x + u * kOrderThreads;
    if (i < padded) sw_lds[i] = v[u];
  }
  __syncthreads();
  // four lanes per slot, each over a quarter of the keys (16-byte reads, interleaved), then a quad sum
  const int gid = blockIdx.x * kOrderThreads + threadIdx.x;
  const int s = gid >> 2, q = gid & 3;
  const int sc = s < slots ? s : slots - 1;
  const int32_t mine = sw_lds[sc];
  const int4* k4 = reinterpret_cast<const int4*>(sw_lds);
  int pos = 0;
#pragma unroll 4
  for (int o = q; o < padded / 4; o += 4) {
    const int4 v = k4[o];
    pos += (v.x < mine) + (v.y < mine) + (v.z < mine) + (v.w < mine);
  }
  pos += __shfl_xor(pos, 1);
  pos += __shfl_xor(pos, 2);
  if (s >= slots || q != 0) return;
  if (shared_early) {
    const int tokens = slots / (top_k + 1), routed = tokens * top_k;
    pos = pos < routed ? pos + (pos < tokens ? pos : tokens) : 2 * (pos - routed) + 1;
  }
  order[pos] = s;
}

constexpr int kTileThreads = 256;
__global__ __launch_bounds__(kTileThreads) void tile_list_kernel(const DgppMoeSegment* __restrict__ segs, int n_segs,
                                                                 int tile_rows, DgppMoeTile* __restrict__ tiles,
                                                                 int32_t* __restrict__ count) {
  __shared__ int s_wave[16];
  int running = 0;
  for (int base = 0; base < n_segs; base += kTileThreads) {
    const int e = base + threadIdx.x;
    const int rows = e < n_segs ? segs[e].rows : 0;
    const int mine = (rows + tile_rows - 1) / tile_rows;
    int total = 0;
    const int excl = block_exclusive_scan(mine, s_wave, &total);
    for (int j = 0; j < mine; ++j) tiles[running + excl + j] = DgppMoeTile{e, j * tile_rows};
    running += total;
  }
  if (threadIdx.x == 0) *count = running;
}

__global__ void compact_segments_kernel(const DgppMoeSegment* __restrict__ input, DgppMoeSegment* __restrict__ output,
                                        int experts, int capacity) {
  __shared__ int s_wave[16];
  const int e = threadIdx.x;
  const int live = (e < experts && input[e].rows > 0) ? 1 : 0;
  int total = 0;
  const int at = block_exclusive_scan(live, s_wave, &total);
  if (live && at < capacity) output[at] = input[e];
  if (e >= total && e < capacity) output[e] = DgppMoeSegment{0, 0, 0};
}

// ---- FP8 -> BF16 bridge ------------------------------------------------------------------------------
template <bool kE8M0>
__global__ void fp8_dequant_kernel(const uint8_t* __restrict__ payload, const void* __restrict__ scales,
                                   uint16_t* __restrict__ out, int64_t rows, int64_t cols, int64_t scale_cols,
                                   int rs, int cs) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  const int64_t n = i / cols, k = i - n * cols;
  const int64_t si = (n >> rs) * scale_cols + (k >> cs);
  float s;
  if (kE8M0) {
    const uint32_t b = static_cast<const uint8_t*>(scales)[si];
    s = b ? bits_f32(b << 23) : bits_f32(0x00400000u);
  } else {
    s = static_cast<const float*>(scales)[si];
  }
  out[i] = f32_to_bf16(e4m3_to_f32(payload[i]) * s);
}

inline unsigned blocks_for(int64_t n) { return static_cast<unsigned>((n + kElemThreads - 1) / kElemThreads); }

}  // namespace

hipError_t run_router_dots(int mode, const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                           float* biased, int tokens, int hidden_dim, int n_experts, hipStream_t stream) {
  const int vec = (hidden_dim % 8 == 0) && ((reinterpret_cast<uintptr_t>(hidden) & 15u) == 0) &&
                  ((reinterpret_cast<uintptr_t>(gate) & 15u) == 0);
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

hipError_t run_router_select(int mode, const float* scores, const float* biased, int32_t* ids, float* weights,
                             int tokens, int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream) {
  const bool softmax = mode == DGPP_ROUTER_SOFTMAX_TOPK;
  const dim3 grid(tokens), block(kWaveSize);
  if (n_experts <= 4 * kWaveSize) {
    if (softmax)
      hipLaunchKernelGGL((router_select_reg_kernel<DGPP_ROUTER_SOFTMAX_TOPK, 4>), grid, block, 0, stream, scores, biased,
                         ids, weights, tokens, n_experts, top_k, scaling, norm_topk);
    else
      hipLaunchKernelGGL((router_select_reg_kernel<DGPP_ROUTER_SIGMOID_BIAS, 4>), grid, block, 0, stream, scores, biased,
                         ids, weights, tokens, n_experts, top_k, scaling, norm_topk);
  } else if (n_experts <= 8 * kWaveSize) {
    if (softmax)
      hipLaunchKernelGGL((router_select_reg_kernel<DGPP_ROUTER_SOFTMAX_TOPK, 8>), grid, block, 0, stream, scores, biased,
                         ids, weights, tokens, n_experts, top_k, scaling, norm_topk);
    else
      hipLaunchKernelGGL((router_select_reg_kernel<DGPP_ROUTER_SIGMOID_BIAS, 8>), grid, block, 0, stream, scores, biased,
                         ids, weights, tokens, n_experts, top_k, scaling, norm_topk);
  } else {
    const size_t lds = 2 * static_cast<size_t>(n_experts) * sizeof(float);
    if (softmax)
      hipLaunchKernelGGL(router_select_kernel<DGPP_ROUTER_SOFTMAX_TOPK>, grid, block, lds, stream, scores, biased, ids,
                         weights, tokens, n_experts, top_k, scaling, norm_topk);
    else
      hipLaunchKernelGGL(router_select_kernel<DGPP_ROUTER_SIGMOID_BIAS>, grid, block, lds, stream, scores, biased, ids,
                         weights, tokens, n_experts, top_k, scaling, norm_topk);
  }
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

hipError_t run_swiglu_clamp(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, float limit,
                            hipStream_t stream) {
  hipLaunchKernelGGL(swiglu_clamp_kernel, dim3(blocks_for(n)), dim3(kElemThreads), 0, stream, gate, up, out, n, limit);
  return hipGetLastError();
}

hipError_t run_gather_rows(const uint16_t* src, const int32_t* rows, uint16_t* dst, int n_rows, int hidden,
                           hipStream_t stream) {
  const bool vec = hidden % 8 == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
  const int unit = vec ? 8 : 1;
  const int per_row = hidden / unit;
  const int64_t units = static_cast<int64_t>(n_rows) * per_row;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks_for(units)), dim3(kElemThreads), 0, stream, src, rows, dst, units,
                     per_row, unit, hidden);
  return hipGetLastError();
}

hipError_t run_accum(float* acc, const float* y, const int32_t* rows, const float* row_w, int n_rows, int hidden,
                     hipStream_t stream) {
  const int64_t n = static_cast<int64_t>(n_rows) * hidden;
  hipLaunchKernelGGL(accum_kernel, dim3(blocks_for(n)), dim3(kElemThreads), 0, stream, acc, y, rows, row_w, n, hidden);
  return hipGetLastError();
}

hipError_t run_round_bf16(uint16_t* out, const float* acc, int64_t n, hipStream_t stream) {
  hipLaunchKernelGGL(round_bf16_kernel, dim3(blocks_for(n)), dim3(kElemThreads), 0, stream, out, acc, n);
  return hipGetLastError();
}

hipError_t run_slot_accum(void* out, int out_f32, int with_shared, const float* contrib, const float* weights,
                          int tokens, int hidden, int top_k, hipStream_t stream) {
  const int64_t n = static_cast<int64_t>(tokens) * hidden;
  const dim3 grid(blocks_for(n)), block(kElemThreads);
  if (with_shared && !out_f32)
    hipLaunchKernelGGL((slot_accum_kernel<true, false>), grid, block, 0, stream, out, contrib, weights, n, hidden, top_k);
  else if (with_shared)
    hipLaunchKernelGGL((slot_accum_kernel<true, true>), grid, block, 0, stream, out, contrib, weights, n, hidden, top_k);
  else if (!out_f32)
    hipLaunchKernelGGL((slot_accum_kernel<false, false>), grid, block, 0, stream, out, contrib, weights, n, hidden, top_k);
  else
    hipLaunchKernelGGL((slot_accum_kernel<false, true>), grid, block, 0, stream, out, contrib, weights, n, hidden, top_k);
  return hipGetLastError();
}

hipError_t run_accum_ordered(void* out, int out_f32, const float* down, size_t down_stride, const int32_t* slot_row,
                             const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens, int top_k,
                             int hidden, hipStream_t stream) {
  const int64_t n = static_cast<int64_t>(tokens) * hidden;
  const dim3 grid(blocks_for(n)), block(kElemThreads);
  if (out_f32)
    hipLaunchKernelGGL(accum_ordered_kernel<true>, grid, block, 0, stream, out, down, down_stride, slot_row, slot_ids,
                       slot_w, shared_row0, tokens, top_k, hidden);
  else
    hipLaunchKernelGGL(accum_ordered_kernel<false>, grid, block, 0, stream, out, down, down_stride, slot_row, slot_ids,
                       slot_w, shared_row0, tokens, top_k, hidden);
  return hipGetLastError();
}

// Plain streaming copy, 16 bytes per lane per step, grid-stride: the calibration workload for
// a profiler's HBM byte counters.
__global__ __launch_bounds__(256) void probe_copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride)
    dst[i] = src[i];
}

hipError_t run_probe_copy(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  const size_t n16 = bytes / 16;
  const size_t want = (n16 + 255) / 256;
  const unsigned blocks = static_cast<unsigned>(want < 1 ? 1 : (want > 16384 ? 16384 : want));
  hipLaunchKernelGGL(probe_copy_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<uint4*>(dst),
                     static_cast<const uint4*>(src), n16);
  return hipGetLastError();
}

hipError_t run_segment(const int32_t* ids, int tokens, int top_k, int n_experts, int32_t* rows, int32_t* slot_row,
                       DgppMoeSegment* segs, hipStream_t stream) {
  hipLaunchKernelGGL(segment_kernel, dim3(n_experts + 1), dim3(kSegThreads), 0, stream, ids, tokens, top_k, n_experts,
                     rows, slot_row, segs);
  return hipGetLastError();
}

hipError_t run_slot_order(const int32_t* ids, int32_t* order, int32_t* runs, int slots, int top_k, int n_experts,
                          int shared_early, hipStream_t stream) {
  if (runs == nullptr && slots > kOrderThreads) {
    const size_t wide_lds = static_cast<size_t>((slots + 3) & ~3) * sizeof(int32_t);
    hipLaunchKernelGGL(slot_order_wide_kernel, dim3((4 * slots + kOrderThreads - 1) / kOrderThreads), dim3(kOrderThreads), wide_lds,
                       stream, ids, order, slots, top_k, n_experts, shared_early);
    return hipGetLastError();
  }
  const int threads = (slots + kWaveSize - 1) / kWaveSize * kWaveSize;
  const size_t lds = (static_cast<size_t>((slots + 3) & ~3) + (runs ? 2 * static_cast<size_t>(slots) : 0)) * sizeof(int32_t);
  hipLaunchKernelGGL(slot_order_kernel, dim3(1), dim3(threads), lds, stream, ids, order, runs, slots, top_k, n_experts,
                     shared_early);
  return hipGetLastError();
}

hipError_t run_tile_list(const DgppMoeSegment* segs, int n_segs, int tile_rows, DgppMoeTile* tiles, int32_t* count,
                         hipStream_t stream) {
  hipLaunchKernelGGL(tile_list_kernel, dim3(1), dim3(kTileThreads), 0, stream, segs, n_segs, tile_rows, tiles, count);
  return hipGetLastError();
}

hipError_t run_compact_segments(const DgppMoeSegment* input, DgppMoeSegment* output, int experts, int capacity,
                                hipStream_t stream) {
  const int threads = (experts + kWaveSize - 1) / kWaveSize * kWaveSize;
  hipLaunchKernelGGL(compact_segments_kernel, dim3(1), dim3(threads), 0, stream, input, output, experts, capacity);
  return hipGetLastError();
}

hipError_t run_fp8_dequant(const uint8_t* payload, const void* scales, int e8m0, uint16_t* out, int64_t rows,
                           int64_t cols, int rs, int cs, hipStream_t stream) {
  const int64_t scale_cols = (cols + (1LL << cs) - 1) >> cs;
  const dim3 grid(blocks_for(rows * cols)), block(kElemThreads);
  if (e8m0)
    hipLaunchKernelGGL(fp8_dequant_kernel<true>, grid, block, 0, stream, payload, scales, out, rows, cols, scale_cols, rs,
                       cs);
  else
    hipLaunchKernelGGL(fp8_dequant_kernel<false>, grid, block, 0, stream, payload, scales, out, rows, cols, scale_cols, rs,
                       cs);
  return hipGetLastError();
}

}  // namespace dgpp_amd
