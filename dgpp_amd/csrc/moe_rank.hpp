// The rank of a decode slot among (expert key, slot) pairs, shared by the router and the grouping kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

namespace dgpp_amd {

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
