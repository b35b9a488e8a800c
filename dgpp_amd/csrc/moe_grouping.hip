// Token -> expert grouping of the MoE path: segments (a stable counting sort), the decode slots' expert order,
// the tile list and the compaction of non-empty segments. Every output is an integer, bit-exact contract.
//
// Reference counterparts: src/models/glm/moe_layer.cpp:634-659 (the host grouping that is the specification),
// src/kernels/glm_moe.cu:465-517 (slot order), :1382-1439 (segmentation), :1553-1569 (tile list);
// src/kernels/minimax.cu:33-50 (segment compaction).
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"
#include "moe_misc.hpp"
#include "moe_rank.hpp"

namespace dgpp_amd {
namespace {

constexpr int kWaveSize = 64;

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

}  // namespace

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

}  // namespace dgpp_amd
