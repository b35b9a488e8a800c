// Small block-level helpers shared by the router and the grouping kernels: an exclusive scan over a block and the
// rank of a decode slot among (expert key, slot) pairs.
#pragma once

#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

namespace dgpp_amd {

// Exclusive prefix sum of one int per thread over a block of up to 1024 threads; *total gets
// the block sum. s_wave needs 16 ints. Ends with a barrier, so s_wave may be reused at once.
__device__ __forceinline__ int block_exclusive_scan(int v, int* s_wave, int* total) {
  const int lane = threadIdx.x & (64 - 1), wave = threadIdx.x >> 6;
  const int n_waves = (blockDim.x + 64 - 1) >> 6;
  int x = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int y = __shfl_up(x, off);
    if (lane >= off) x += y;
  }
  if (lane == 64 - 1) s_wave[wave] = x;
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

}  // namespace dgpp_amd
