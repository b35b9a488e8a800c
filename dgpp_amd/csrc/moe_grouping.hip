// Token -> expert grouping of the MoE path: segments (a stable counting sort), the decode slots' expert order,
// the tile list and the compaction of non-empty segments. Every output is an integer, bit-exact contract.
//
// What each output must hold is fixed by the reference: src/models/glm/moe_layer.cpp:634-659 (the host grouping that is
// the specification), src/kernels/glm_moe.cu:465-517 (slot order, runs, group list), :1382-1439 (segmentation),
// :1553-1569 (tile list); src/kernels/minimax.cu:33-50 (segment compaction). How it is computed is this chip's:
// wavefront ballots with mbcnt prefix counts, DPP prefix sums, scalar-side running totals.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"
#include "moe_misc.hpp"
#include "moe_rank.hpp"

namespace dgpp_amd {
namespace {

constexpr int kWaveSize = 64;

// ---- wavefront primitives ------------------------------------------------------------------------
// How many lanes below this one have their bit set in a ballot.
__device__ __forceinline__ int lanes_below(unsigned long long mask) {
  return static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                                    __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u)));
}
template <int kCtrl, int kRowMask>
__device__ __forceinline__ int dpp_take(int v) {   // lanes the move does not reach read 0
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, kRowMask, 0xF, false);
}
// Inclusive prefix sum over the wavefront: four shifts inside each row of sixteen lanes, then the two row
// broadcasts that carry a row's total into the rows after it.
__device__ __forceinline__ int wave_prefix_incl(int v) {
  v += dpp_take<0x111, 0xF>(v);   // row_shr:1
  v += dpp_take<0x112, 0xF>(v);   // row_shr:2
  v += dpp_take<0x114, 0xF>(v);   // row_shr:4
  v += dpp_take<0x118, 0xF>(v);   // row_shr:8
  v += dpp_take<0x142, 0xA>(v);   // row_bcast:15 into rows 1 and 3
  v += dpp_take<0x143, 0xC>(v);   // row_bcast:31 into rows 2 and 3
  return v;
}

// ---- grouping ------------------------------------------------------------------------------------
// The host path's stable counting sort (src/models/glm/moe_layer.cpp:634-659) with ONE WAVEFRONT per expert
// and no LDS, barrier or atomic: the wavefront reads the routed ids sixty-four at a time; two ballots per read
// count, on the scalar side, the ids that sort before its expert (its segment's first row) and its own (the
// segment's length). A second walk places the matches in (token, slot) order: a match's row is the segment's
// rows placed so far plus the matching lanes below it (mbcnt of the ballot). One launch; the wavefront after the
// last expert writes the shared segment.
constexpr int kSegWaves = 4;
__global__ __launch_bounds__(kSegWaves * kWaveSize) void segment_kernel(const int32_t* __restrict__ ids, int tokens, int K,
                                                                         int E, int32_t* __restrict__ rows,
                                                                         int32_t* __restrict__ slot_row,
                                                                         DgppMoeSegment* __restrict__ segs) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int e = blockIdx.x * kSegWaves + (threadIdx.x >> 6);
  if (e > E) return;
  const int tk = tokens * K;
  if (e == E) {  // the shared expert: every token once more, after the routed rows
    for (int t = lane; t < tokens; t += kWaveSize) rows[tk + t] = t;
    if (lane == 0) segs[E] = DgppMoeSegment{tk, tokens, E};
    return;
  }
  int before = 0, own = 0;
  for (int first = 0; first < tk; first += kWaveSize) {
    const int i = first + lane;
    const int id = i < tk ? ids[i] : INT_MAX;
    before += __builtin_popcountll(__builtin_amdgcn_ballot_w64(id < e));
    own += __builtin_popcountll(__builtin_amdgcn_ballot_w64(id == e));
  }
  if (lane == 0) segs[e] = DgppMoeSegment{before, own, e};
  if (own == 0) return;
  int placed = before;
  for (int first = 0; first < tk && placed < before + own; first += kWaveSize) {
    const int i = first + lane;
    const bool hit = i < tk && ids[i] == e;
    const unsigned long long hits = __builtin_amdgcn_ballot_w64(hit);
    if (hit) {
      const int at = placed + lanes_below(hits);
      rows[at] = i / K;
      slot_row[i] = at;
    }
    placed += __builtin_popcountll(hits);
  }
}

// One block, one thread per slot: rank by (key, slot), key = expert id or E for the shared slot. With `runs`: the
// length of every run of equal experts at its first position (0 elsewhere) and, behind it, the list of 64-row
// groups of the runs longer than a 16-row tile (src/kernels/glm_moe.cu:465-517 defines both). Run starts are found
// by ballot; a run's length is the distance to the next start, read off the ballots (this wavefront's mask above
// the lane, else the first set bit of a later wavefront's); a run's first list entry is an exclusive prefix sum of
// the group counts (wavefront scan, wavefront totals through LDS).
__global__ void slot_order_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ order,
                                  int32_t* __restrict__ runs, int slots, int top_k, int n_experts,
                                  int shared_early) {
  extern __shared__ __align__(16) int32_t so_lds[];  // keys [slots padded to 4]; with runs: sorted [slots]
  __shared__ unsigned long long s_starts[16];
  __shared__ int s_groups[16];
  const int padded = (slots + 3) & ~3;
  int32_t* keys = so_lds;
  int32_t* sorted = keys + padded;
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
  const int lane = s & (kWaveSize - 1), wave = s >> 6, n_waves = static_cast<int>(blockDim.x) >> 6;
  const bool starts_run = s < slots && (s == 0 || sorted[s - 1] != sorted[s]);
  const unsigned long long mask = __builtin_amdgcn_ballot_w64(starts_run);
  if (lane == 0) s_starts[wave] = mask;
  __syncthreads();
  int next = slots;   // the position of the next run's start
  {
    const unsigned long long above = lane < kWaveSize - 1 ? mask >> (lane + 1) : 0ull;
    if (above != 0ull) {
      next = s + 1 + __builtin_ctzll(above);
    } else {
      for (int w = wave + 1; w < n_waves; ++w) {
        const unsigned long long m = s_starts[w];
        if (m != 0ull) {
          next = w * kWaveSize + __builtin_ctzll(m);
          break;
        }
      }
    }
  }
  const int len = starts_run ? next - s : 0;
  const int n_groups = len > kTileRows ? (len + kGroupRows - 1) / kGroupRows : 0;
  if (s < slots) runs[s] = len;
  const int upto = wave_prefix_incl(n_groups);
  if (lane == kWaveSize - 1) s_groups[wave] = upto;
  __syncthreads();
  int first_entry = upto - n_groups, listed = 0;
  for (int w = 0; w < n_waves; ++w) {
    const int c = s_groups[w];
    if (w < wave) first_entry += c;
    listed += c;
  }
  int32_t* list = runs + slots;
  for (int g = 0; g < n_groups; ++g) {
    const int r0 = g * kGroupRows;
    list[first_entry + g] = (s + r0) | (min(kGroupRows, len - r0) << 16);
  }
  const int capacity = slots / (kTileRows + 1) + 1;   // the list's entries beyond the groups read -1
  for (int i = listed + s; i < capacity; i += static_cast<int>(blockDim.x)) list[i] = -1;
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

// The (segment, first row) tiles of every segment, in segment order, and their count: ONE wavefront walks the
// segments sixty-four at a time; a segment's first tile is the tiles emitted so far plus the wavefront prefix sum of
// the tile counts below its lane (no LDS, no barrier), and each lane writes its own segment's tiles.
__global__ __launch_bounds__(kWaveSize) void tile_list_kernel(const DgppMoeSegment* __restrict__ segs, int n_segs,
                                                               int tile_rows, DgppMoeTile* __restrict__ tiles,
                                                               int32_t* __restrict__ count) {
  const int lane = threadIdx.x;
  int emitted = 0;
  for (int first = 0; first < n_segs; first += kWaveSize) {
    const int seg = first + lane;
    const int n_tiles = seg < n_segs ? (segs[seg].rows + tile_rows - 1) / tile_rows : 0;
    const int upto = wave_prefix_incl(n_tiles);
    DgppMoeTile* out = tiles + emitted + upto - n_tiles;
    for (int j = 0; j < n_tiles; ++j) out[j] = DgppMoeTile{seg, j * tile_rows};
    emitted += __builtin_amdgcn_readlane(upto, kWaveSize - 1);
  }
  if (lane == 0) *count = emitted;
}

// Stable compaction of the non-empty segments (src/kernels/minimax.cu:33-50): a live segment's place is the live
// lanes below it in its wavefront's ballot plus the live counts of the wavefronts before; entries past the live
// ones read zero.
__global__ void compact_segments_kernel(const DgppMoeSegment* __restrict__ input, DgppMoeSegment* __restrict__ output,
                                        int experts, int capacity) {
  __shared__ int s_live[16];
  const int e = threadIdx.x, lane = e & (kWaveSize - 1), wave = e >> 6, n_waves = static_cast<int>(blockDim.x) >> 6;
  const bool live = e < experts && input[e].rows > 0;
  const unsigned long long mask = __builtin_amdgcn_ballot_w64(live);
  if (lane == 0) s_live[wave] = __builtin_popcountll(mask);
  __syncthreads();
  int at = lanes_below(mask), total = 0;
  for (int w = 0; w < n_waves; ++w) {
    const int c = s_live[w];
    if (w < wave) at += c;
    total += c;
  }
  if (live && at < capacity) output[at] = input[e];
  if (e >= total && e < capacity) output[e] = DgppMoeSegment{0, 0, 0};
}

}  // namespace

hipError_t run_segment(const int32_t* ids, int tokens, int top_k, int n_experts, int32_t* rows, int32_t* slot_row,
                       DgppMoeSegment* segs, hipStream_t stream) {
  hipLaunchKernelGGL(segment_kernel, dim3((n_experts + 1 + kSegWaves - 1) / kSegWaves), dim3(kSegWaves * kWaveSize), 0, stream,
                     ids, tokens, top_k, n_experts, rows, slot_row, segs);
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
  const size_t lds = (static_cast<size_t>((slots + 3) & ~3) + (runs ? static_cast<size_t>(slots) : 0)) * sizeof(int32_t);
  hipLaunchKernelGGL(slot_order_kernel, dim3(1), dim3(threads), lds, stream, ids, order, runs, slots, top_k, n_experts,
                     shared_early);
  return hipGetLastError();
}

hipError_t run_tile_list(const DgppMoeSegment* segs, int n_segs, int tile_rows, DgppMoeTile* tiles, int32_t* count,
                         hipStream_t stream) {
  hipLaunchKernelGGL(tile_list_kernel, dim3(1), dim3(kWaveSize), 0, stream, segs, n_segs, tile_rows, tiles, count);
  return hipGetLastError();
}

hipError_t run_compact_segments(const DgppMoeSegment* input, DgppMoeSegment* output, int experts, int capacity,
                                hipStream_t stream) {
  const int threads = (experts + kWaveSize - 1) / kWaveSize * kWaveSize;
  hipLaunchKernelGGL(compact_segments_kernel, dim3(1), dim3(threads), 0, stream, input, output, experts, capacity);
  return hipGetLastError();
}

}  // namespace dgpp_amd
