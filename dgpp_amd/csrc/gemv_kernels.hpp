// Kernels built on the GEMV core: the dense projection, the MoE decode-slot kernels (fused
// gate/up + SwiGLU, down) and the grouped (segment-major) twin. One template per kernel,
// instantiated per weight format in gemv_fp8.hip / gemv_fp4.hip.
//
// Reference counterparts: src/kernels/fp4_gemv.cu:16-95, src/kernels/scale_gemm.cu:168-197,
// src/kernels/glm_moe.cu:572-667 (FP8 slot kernels), :1863-1953 and :2061-2144 (FP4 slot kernels),
// :999-1059 and :2149-2195 (grouped kernels).
#pragma once

#include <type_traits>

#include "../../include/dgpp_amd.h"
#include "gemv_core.hpp"

namespace dgpp_amd {

// Every GEMV kernel is compiled for at least this many resident wavefronts per SIMD (a cap of 128
// VGPRs): the streams are latency-bound, and the compiler otherwise trades occupancy for hoisting
// every decode of a pass ahead of the first dot.
#ifndef DGPP_MIN_WAVES_PER_SIMD
#define DGPP_MIN_WAVES_PER_SIMD 2
#endif
constexpr int kMinWavesPerSimd = DGPP_MIN_WAVES_PER_SIMD;

// ---- epilogues ------------------------------------------------------------------------------
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// SwiGLU on the bf16-rounded dots with the reference's rounding points
// (src/kernels/glm_moe.cu:659-666): gate clamped above only, up on both sides.
__device__ __forceinline__ uint16_t swiglu_bf16(float gate_dot, float up_dot, float limit) {
  float g = bf16_to_f32(f32_to_bf16(gate_dot));
  float u = bf16_to_f32(f32_to_bf16(up_dot));
  if (g > limit) g = limit;
  u = fminf(fmaxf(u, -limit), limit);
  const uint16_t t = f32_to_bf16(g * sigmoid_f32(g));
  return f32_to_bf16(bf16_to_f32(t) * u);
}

template <int FMT>
__device__ __forceinline__ float finish_dot(float acc, float divisor) {
  if constexpr (FMT == kFmtNvfp4) return acc / divisor;  // one correctly rounded division
  return acc;
}

template <int FMT>
__device__ __forceinline__ float load_divisor(const float* global) {
  if constexpr (FMT == kFmtNvfp4) return *global;
  return 1.0f;
}

// The row geometry every launcher uses for a k-wide row of format FMT (one function, so the slot,
// grouped and dense forms agree bit for bit).
template <int FMT>
inline RowGeom geom_for(int k) {
  const int prefer = tune_get(kTunePreferP);
  return row_geom(k / FmtTraits<FMT>::kElemsPerChunk, prefer > 0 ? prefer : 4);
}

// rows a block covers: waves x rows-per-wave x steps
__host__ __device__ inline int block_rows(const RowGeom& g, int steps) {
  return kWavesPerBlock * (kWave >> g.l2) * steps;
}

// ---- dense projection -------------------------------------------------------------------------
struct DenseArgs {
  const uint16_t* act;
  size_t act_stride;
  MatRef mat;
  const float* global;   // NVFP4 device global
  void* out;
  size_t out_stride;
  int out_f32;
  int m, n, k;
};

template <int FMT, int MAXR, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void gemv_dense_kernel(DenseArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  stage_activations<FMT>(a.act, a.act_stride, a.m, a.k, lds);
  __syncthreads();
  const float divisor = load_divisor<FMT>(a.global);
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  int row0 = blockIdx.x * block_rows(g, steps) + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const LaneRow lr = lane_row<FMT>(a.mat, row0, a.n, a.k, g.l2);
    float acc[MAXR];
    row_dots<FMT, MAXR, NB>(lr, g, a.mat.cs, lds, chunks, a.m, acc);
    if (lr.li == 0 && lr.row < a.n) {
#pragma unroll
      for (int r = 0; r < MAXR; ++r) {
        if (r < a.m) {
          const float v = finish_dot<FMT>(acc[r], divisor);
          const size_t at = static_cast<size_t>(r) * a.out_stride + lr.row;
          if (a.out_f32)
            static_cast<float*>(a.out)[at] = v;
          else
            static_cast<uint16_t*>(a.out)[at] = f32_to_bf16(v);
        }
      }
    }
  }
}

// ---- MoE decode slots ----------------------------------------------------------------------------
// Slot layout (src/kernels/glm_moe_launch.hpp:216-226): slot = t * (top_k + 1) + j, j < top_k the
// token's j-th routed expert (ascending id), j == top_k the shared expert.
struct SlotArgs {
  const uint16_t* x;        // gate/up: token rows; down: slot activation rows
  size_t x_stride;
  const int32_t* ids;
  const int32_t* order;     // nullable: blockIdx.y -> logical slot
  const DgppMoeExpertView* views;
  MatRef sh[2];             // shared expert matrices given as launch arguments (FP8)
  void* out;                // gate/up: bf16 act [slots, out_stride]; down: f32 [slots, out_stride]
  int out_stride;
  int n, k;                 // the dims of the slots this launch computes
  int slots, top_k;
  float limit;
  int want_shared;          // 0: routed slots, 1: shared slots (others exit)
  int shared_view_base;     // >= 0: shared matrices come from views[base + which]
  int debug_nomath;         // bench probe: loads only
};

template <int FMT>
__device__ __forceinline__ MatRef mat_of_view(const DgppMoeExpertView& v, const float** global) {
  MatRef m;
  m.payload = v.payload;
  if constexpr (FMT == kFmtFp8F32) {
    m.scales = v.scales;
    m.rs = v.scale_shift_rows;
    m.cs = v.scale_shift_cols;
    *global = nullptr;
  } else {
    m.scales = v.fp4_scales;
    m.rs = 0;
    m.cs = 0;
    *global = v.fp4_global;
  }
  m.divisor = 1.0f;
  return m;
}

// Resolves the slot of this block; false when the block has nothing to do.
__device__ __forceinline__ bool resolve_slot(const SlotArgs& a, int& slot, int& token, int& view_base) {
  if (static_cast<int>(blockIdx.y) >= a.slots) return false;
  slot = a.order ? a.order[blockIdx.y] : static_cast<int>(blockIdx.y);
  token = slot / (a.top_k + 1);
  const int j = slot - token * (a.top_k + 1);
  const bool shared = j == a.top_k;
  if (shared != (a.want_shared != 0)) return false;
  view_base = shared ? a.shared_view_base : a.ids[static_cast<size_t>(token) * a.top_k + j] * 3;
  return true;
}

template <int FMT, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_gate_up_kernel(SlotArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  int slot, token, base;
  if (!resolve_slot(a, slot, token, base)) return;
  const int rows_per_block = block_rows(g, steps);
  if (static_cast<int>(blockIdx.x) * rows_per_block >= a.n) return;
  MatRef mg, mu;
  const float *gg = nullptr, *gu = nullptr;
  if (base >= 0) {
    mg = mat_of_view<FMT>(a.views[base + 0], &gg);
    mu = mat_of_view<FMT>(a.views[base + 1], &gu);
  } else {
    mg = a.sh[0];
    mu = a.sh[1];
  }
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  stage_activations<FMT>(a.x + static_cast<size_t>(token) * a.x_stride, a.x_stride, 1, a.k, lds);
  __syncthreads();
  const float dg = load_divisor<FMT>(gg), du = load_divisor<FMT>(gu);
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  uint16_t* act_row = static_cast<uint16_t*>(a.out) + static_cast<size_t>(slot) * a.out_stride;
  int row0 = blockIdx.x * rows_per_block + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const LaneRow lg = lane_row<FMT>(mg, row0, a.n, a.k, g.l2);
    const LaneRow lu = lane_row<FMT>(mu, row0, a.n, a.k, g.l2);
    float ag, au;
    row_dots_pair<FMT, NB>(lg, lu, g, mg.cs, mu.cs, lds, chunks, ag, au);
    if (lg.li == 0 && lg.row < a.n)
      act_row[lg.row] = swiglu_bf16(finish_dot<FMT>(ag, dg), finish_dot<FMT>(au, du), a.limit);
  }
}

template <int FMT, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_down_kernel(SlotArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  int slot, token, base;
  if (!resolve_slot(a, slot, token, base)) return;
  const int rows_per_block = block_rows(g, steps);
  if (static_cast<int>(blockIdx.x) * rows_per_block >= a.n) return;
  MatRef md;
  const float* gd = nullptr;
  if (base >= 0)
    md = mat_of_view<FMT>(a.views[base + 2], &gd);
  else
    md = a.sh[0];
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  // The down projection consumes this slot's own activation row.
  stage_activations<FMT>(a.x + static_cast<size_t>(slot) * a.x_stride, a.x_stride, 1, a.k, lds);
  __syncthreads();
  const float dd = load_divisor<FMT>(gd);
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  float* out_row = static_cast<float*>(a.out) + static_cast<size_t>(slot) * a.out_stride;
  int row0 = blockIdx.x * rows_per_block + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const LaneRow lr = lane_row<FMT>(md, row0, a.n, a.k, g.l2);
    float acc[1];
    row_dots<FMT, 1, NB>(lr, g, md.cs, lds, chunks, 1, acc);
    if (lr.li == 0 && lr.row < a.n) out_row[lr.row] = finish_dot<FMT>(acc[0], dd);
  }
}

// ---- decode slots, register-resident activations ---------------------------------------------------
// The slot kernels' fast form when a row fits ONE pass (P == NB chunks per lane) and the activation
// row is 16-byte aligned: a lane's chunk columns are the same for every weight row it visits, so it
// loads its own slice of the activation row into registers ONCE (straight from global memory: no
// LDS, no barrier) and then streams weight rows: both matrices of a step are issued together and
// the next step's loads are issued before the current step is consumed, so a lane keeps up to
// 4 * NB 16-byte loads in flight. The per-(row) arithmetic — chunk order per lane, dot2 order,
// butterfly — is exactly the LDS form's: the two are bitwise twins.
template <int FMT, int NB>
struct XSlice {
  uint4 v[NB * FmtTraits<FMT>::kPieces];
};
template <int FMT, int NB>
__device__ __forceinline__ void load_x_slice(const uint16_t* __restrict__ x, int li, int l2, XSlice<FMT, NB>& xs) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int c = (i << l2) + li;
#pragma unroll
    for (int q = 0; q < kPieces; ++q)
      xs.v[i * kPieces + q] = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(c * kPieces + q) * 8);
  }
}
template <int FMT, int NB>
__device__ __forceinline__ float dot_pass_reg(const ChunkRegs (&regs)[NB], const XSlice<FMT, NB>& xs, int l2) {
  float acc[1] = {0.f};
#pragma unroll
  for (int i = 0; i < NB; ++i)
    consume_chunk<FMT, 1>(regs[i], XReg<FMT>{xs.v + i * FmtTraits<FMT>::kPieces}, 1, acc);
  return group_sum(acc[0], l2);
}

template <int FMT, int NB, bool PREFETCH>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_gate_up_reg_kernel(SlotArgs a, RowGeom g, int steps) {
  int slot, token, base;
  if (!resolve_slot(a, slot, token, base)) return;
  const int rows_per_block = block_rows(g, steps);
  if (static_cast<int>(blockIdx.x) * rows_per_block >= a.n) return;
  MatRef mg, mu;
  const float *gg = nullptr, *gu = nullptr;
  if (base >= 0) {
    mg = mat_of_view<FMT>(a.views[base + 0], &gg);
    mu = mat_of_view<FMT>(a.views[base + 1], &gu);
  } else {
    mg = a.sh[0];
    mu = a.sh[1];
  }
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  const int stride = kWavesPerBlock * rpw;
  int row0 = blockIdx.x * rows_per_block + wave * rpw;
  if (row0 >= a.n) return;
  // The first step's weight loads go out before anything else (the longest latency of the block).
  LaneRow lg = lane_row<FMT>(mg, row0, a.n, a.k, g.l2);
  LaneRow lu = lane_row<FMT>(mu, row0, a.n, a.k, g.l2);
  ChunkRegs cg[NB], cu[NB];
  issue_pass<FMT, NB>(lg, 0, g.l2, mg.cs, cg);
  issue_pass<FMT, NB>(lu, 0, g.l2, mu.cs, cu);
  XSlice<FMT, NB> xs;
  load_x_slice<FMT, NB>(a.x + static_cast<size_t>(token) * a.x_stride, lg.li, g.l2, xs);
  const float dg = load_divisor<FMT>(gg), du = load_divisor<FMT>(gu);
  uint16_t* act_row = static_cast<uint16_t*>(a.out) + static_cast<size_t>(slot) * a.out_stride;
  for (int s = 0; s < steps; ++s) {
    const int next0 = row0 + stride;
    const bool has_next = s + 1 < steps && next0 < a.n;
    ChunkRegs ng[NB], nu[NB];
    LaneRow lgn = lg, lun = lu;
    if (has_next) {
      lgn = lane_row<FMT>(mg, next0, a.n, a.k, g.l2);
      lun = lane_row<FMT>(mu, next0, a.n, a.k, g.l2);
      if constexpr (PREFETCH) {
        issue_pass<FMT, NB>(lgn, 0, g.l2, mg.cs, ng);
        issue_pass<FMT, NB>(lun, 0, g.l2, mu.cs, nu);
      }
    }
    float ag, au;
    if (a.debug_nomath) {
      uint32_t t = 0;
#pragma unroll
      for (int i = 0; i < NB; ++i) t ^= cg[i].w.x ^ cg[i].w.y ^ cg[i].w.z ^ cg[i].w.w ^ cu[i].w.x ^ cu[i].w.y ^ cu[i].w.z ^ cu[i].w.w ^ cg[i].s ^ cu[i].s;
      ag = au = bits_f32(t & 0x3FFFFFFFu);
    } else {
      ag = dot_pass_reg<FMT, NB>(cg, xs, g.l2);
      au = dot_pass_reg<FMT, NB>(cu, xs, g.l2);
    }
    if (lg.li == 0 && lg.row < a.n)
      act_row[lg.row] = swiglu_bf16(finish_dot<FMT>(ag, dg), finish_dot<FMT>(au, du), a.limit);
    if (!has_next) break;
    if constexpr (PREFETCH) {
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        cg[i] = ng[i];
        cu[i] = nu[i];
      }
    } else {
      issue_pass<FMT, NB>(lgn, 0, g.l2, mg.cs, cg);
      issue_pass<FMT, NB>(lun, 0, g.l2, mu.cs, cu);
    }
    lg = lgn;
    lu = lun;
    row0 = next0;
  }
}

template <int FMT, int NB, bool PREFETCH>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_down_reg_kernel(SlotArgs a, RowGeom g, int steps) {
  int slot, token, base;
  if (!resolve_slot(a, slot, token, base)) return;
  const int rows_per_block = block_rows(g, steps);
  if (static_cast<int>(blockIdx.x) * rows_per_block >= a.n) return;
  MatRef md;
  const float* gd = nullptr;
  if (base >= 0)
    md = mat_of_view<FMT>(a.views[base + 2], &gd);
  else
    md = a.sh[0];
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  const int stride = kWavesPerBlock * rpw;
  int row0 = blockIdx.x * rows_per_block + wave * rpw;
  if (row0 >= a.n) return;
  LaneRow lr = lane_row<FMT>(md, row0, a.n, a.k, g.l2);
  ChunkRegs cur[NB];
  issue_pass<FMT, NB>(lr, 0, g.l2, md.cs, cur);
  XSlice<FMT, NB> xs;
  load_x_slice<FMT, NB>(a.x + static_cast<size_t>(slot) * a.x_stride, lr.li, g.l2, xs);
  const float dd = load_divisor<FMT>(gd);
  float* out_row = static_cast<float*>(a.out) + static_cast<size_t>(slot) * a.out_stride;
  for (int s = 0; s < steps; ++s) {
    const int next0 = row0 + stride;
    const bool has_next = s + 1 < steps && next0 < a.n;
    ChunkRegs nxt[NB];
    LaneRow ln = lr;
    if (has_next) {
      ln = lane_row<FMT>(md, next0, a.n, a.k, g.l2);
      if constexpr (PREFETCH) issue_pass<FMT, NB>(ln, 0, g.l2, md.cs, nxt);
    }
    const float acc = dot_pass_reg<FMT, NB>(cur, xs, g.l2);
    if (lr.li == 0 && lr.row < a.n) out_row[lr.row] = finish_dot<FMT>(acc, dd);
    if (!has_next) break;
    if constexpr (PREFETCH) {
#pragma unroll
      for (int i = 0; i < NB; ++i) cur[i] = nxt[i];
    } else {
      issue_pass<FMT, NB>(ln, 0, g.l2, md.cs, cur);
    }
    lr = ln;
    row0 = next0;
  }
}

// The register form applies when the whole row is one pass and the lane's activation slice stays
// within 64 registers.
template <int FMT>
inline bool slot_reg_form_ok(const RowGeom& g, const SlotArgs& a) {
  const int xregs = g.P * FmtTraits<FMT>::kPieces * 4;
  return g.P == g.nb && xregs <= 64 && ((reinterpret_cast<uintptr_t>(a.x) & 15u) == 0) && ((a.x_stride & 7u) == 0);
}

// ---- grouped (segment-major) twin ------------------------------------------------------------------
struct GroupedArgs {
  const uint16_t* act;
  size_t act_stride;
  const DgppMoeSegment* segs;
  const DgppMoeExpertView* views;
  int which;
  void* out;
  size_t out_stride;
  int out_f32;
  int n, k;
  int rows_per_block;  // segment rows per z block
  int group_rows;      // activation rows staged per pass (<= kMaxActRows)
};

template <int FMT, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void grouped_gemv_kernel(GroupedArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  const DgppMoeSegment seg = a.segs[blockIdx.y];
  const int z0 = static_cast<int>(blockIdx.z) * a.rows_per_block;
  if (z0 >= seg.rows) return;
  const int z1 = min(seg.rows, z0 + a.rows_per_block);
  const float* gp = nullptr;
  const MatRef mat = mat_of_view<FMT>(a.views[seg.expert * 3 + a.which], &gp);
  const float divisor = load_divisor<FMT>(gp);
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  for (int g0 = z0; g0 < z1; g0 += a.group_rows) {
    const int m = min(a.group_rows, z1 - g0);
    if (g0 > z0) __syncthreads();  // the previous group is done reading the staged rows
    stage_activations<FMT>(a.act + static_cast<size_t>(seg.row0 + g0) * a.act_stride, a.act_stride, m, a.k, lds);
    __syncthreads();
    int row0 = blockIdx.x * block_rows(g, steps) + wave * rpw;
    for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
      if (row0 >= a.n) break;
      const LaneRow lr = lane_row<FMT>(mat, row0, a.n, a.k, g.l2);
      float acc[kMaxActRows];
      row_dots<FMT, kMaxActRows, NB>(lr, g, mat.cs, lds, chunks, m, acc);
      if (lr.li == 0 && lr.row < a.n) {
#pragma unroll
        for (int r = 0; r < kMaxActRows; ++r) {
          if (r < m) {
            const float v = finish_dot<FMT>(acc[r], divisor);
            const size_t at = static_cast<size_t>(seg.row0 + g0 + r) * a.out_stride + lr.row;
            if (a.out_f32)
              static_cast<float*>(a.out)[at] = v;
            else
              static_cast<uint16_t*>(a.out)[at] = f32_to_bf16(v);
          }
        }
      }
    }
  }
}

// ---- host launch helpers (defined per format in gemv_fp8.hip / gemv_fp4.hip) ---------------------------
// Elements per chunk by format, and the LDS bytes `rows` staged activation rows take.
inline int elems_per_chunk(int fmt) { return fmt >= kFmtNvfp4 ? 32 : 16; }
inline size_t stage_bytes(int rows, int k) { return static_cast<size_t>(rows) * static_cast<size_t>(k) * 2; }

// Row steps per block: enough blocks to fill the 256 CUs several times over while amortising
// the activation staging of a block over more weight rows on large problems.
inline int pick_steps(long long block_steps_total) {
  long long s = (block_steps_total + 4095) / 4096;
  if (s < 1) s = 1;
  if (s > 8) s = 8;
  return static_cast<int>(s);
}

hipError_t launch_dense(int fmt, const DenseArgs& a, hipStream_t stream);
hipError_t launch_slot_gate_up(int fmt, const SlotArgs& a, hipStream_t stream);
hipError_t launch_slot_down(int fmt, const SlotArgs& a, hipStream_t stream);
hipError_t launch_grouped(int fmt, const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream);

// Per-format implementations.
template <int FMT> hipError_t launch_dense_fmt(const DenseArgs& a, hipStream_t stream);
template <int FMT> hipError_t launch_slot_gate_up_fmt(const SlotArgs& a, hipStream_t stream);
template <int FMT> hipError_t launch_slot_down_fmt(const SlotArgs& a, hipStream_t stream);
template <int FMT> hipError_t launch_grouped_fmt(const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream);

// Raises a kernel's dynamic LDS ceiling (once per kernel) when a launch needs more than the
// default 64 KB; gfx950 offers 160 KB per workgroup.
hipError_t ensure_lds_impl(const void* kernel, size_t bytes);
template <class K>
inline hipError_t ensure_lds(K kernel, size_t bytes) {
  if (bytes <= kDefaultLdsBytes) return hipSuccess;
  return ensure_lds_impl(reinterpret_cast<const void*>(kernel), bytes);
}
// Activation rows one launch may stage for a k-wide row (at most kMaxActRows).
inline int max_stage_rows(int k) {
  const size_t per_row = static_cast<size_t>(k) * 2;
  const size_t fit = per_row ? kMaxLdsBytes / per_row : kMaxActRows;
  return static_cast<int>(fit < 1 ? 1 : (fit > kMaxActRows ? kMaxActRows : fit));
}

// The bodies, included by the per-format translation units.
#ifdef DGPP_GEMV_IMPL
template <int FMT>
hipError_t launch_dense_fmt(const DenseArgs& a, hipStream_t stream) {
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long block_steps = (a.n + rows_per_step - 1) / rows_per_step;
  const int steps = pick_steps(block_steps);
  const dim3 grid(static_cast<unsigned>((block_steps + steps - 1) / steps));
  const size_t lds = stage_bytes(a.m, a.k);
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    auto go = [&](auto rc) {
      constexpr int MAXR = decltype(rc)::value;
      auto kern = gemv_dense_kernel<FMT, MAXR, NB>;
      err = ensure_lds(kern, lds);
      if (err != hipSuccess) return;
      hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g, steps);
    };
    if (a.m == 1) go(std::integral_constant<int, 1>{});
    else if (a.m == 2) go(std::integral_constant<int, 2>{});
    else if (a.m <= 4) go(std::integral_constant<int, 4>{});
    else go(std::integral_constant<int, 8>{});
  });
  return err != hipSuccess ? err : hipGetLastError();
}

// Row steps per block of a slot launch: about four resident rounds of blocks over the 256 CUs.
inline int pick_slot_steps(long long block_steps_total) {
  long long s = (block_steps_total + 2047) / 2048;
  if (s < 1) s = 1;
  if (s > 16) s = 16;
  return static_cast<int>(s);
}

template <int FMT>
hipError_t launch_slot_gate_up_fmt(const SlotArgs& a, hipStream_t stream) {
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long per_slot = (a.n + rows_per_step - 1) / rows_per_step;
  const int form = tune_get(kTuneSlotForm);   // 0 auto, 1 LDS, 2 registers + prefetch, 3 registers
  const_cast<SlotArgs&>(a).debug_nomath = tune_get(3);
  const bool reg = form >= 2 && slot_reg_form_ok<FMT>(g, a);
  int steps = reg ? pick_slot_steps(per_slot * a.slots) : pick_steps(per_slot * a.slots);
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  const dim3 grid(static_cast<unsigned>((per_slot + steps - 1) / steps), static_cast<unsigned>(a.slots));
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    if constexpr (NB * FmtTraits<FMT>::kPieces * 4 <= 64) {
      if (reg && form == 2) {
        hipLaunchKernelGGL((slot_gate_up_reg_kernel<FMT, NB, true>), grid, dim3(kBlockThreads), 0, stream, a, g, steps);
        return;
      }
      if (reg) {
        hipLaunchKernelGGL((slot_gate_up_reg_kernel<FMT, NB, false>), grid, dim3(kBlockThreads), 0, stream, a, g, steps);
        return;
      }
    }
    hipLaunchKernelGGL((slot_gate_up_kernel<FMT, NB>), grid, dim3(kBlockThreads), stage_bytes(1, a.k), stream, a, g, steps);
  });
  return hipGetLastError();
}

template <int FMT>
hipError_t launch_slot_down_fmt(const SlotArgs& a, hipStream_t stream) {
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long per_slot = (a.n + rows_per_step - 1) / rows_per_step;
  const int form = tune_get(kTuneSlotForm);
  const bool reg = form >= 2 && slot_reg_form_ok<FMT>(g, a);
  int steps = reg ? pick_slot_steps(per_slot * a.slots) : pick_steps(per_slot * a.slots);
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  const dim3 grid(static_cast<unsigned>((per_slot + steps - 1) / steps), static_cast<unsigned>(a.slots));
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    if constexpr (NB * FmtTraits<FMT>::kPieces * 4 <= 64) {
      if (reg && form == 2) {
        hipLaunchKernelGGL((slot_down_reg_kernel<FMT, NB, true>), grid, dim3(kBlockThreads), 0, stream, a, g, steps);
        return;
      }
      if (reg) {
        hipLaunchKernelGGL((slot_down_reg_kernel<FMT, NB, false>), grid, dim3(kBlockThreads), 0, stream, a, g, steps);
        return;
      }
    }
    hipLaunchKernelGGL((slot_down_kernel<FMT, NB>), grid, dim3(kBlockThreads), stage_bytes(1, a.k), stream, a, g, steps);
  });
  return hipGetLastError();
}

template <int FMT>
hipError_t launch_grouped_fmt(const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream) {
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long per_seg = (a.n + rows_per_step - 1) / rows_per_step;
  const int steps = pick_steps(per_seg * n_segs);
  const dim3 grid(static_cast<unsigned>((per_seg + steps - 1) / steps), static_cast<unsigned>(n_segs),
                  static_cast<unsigned>(z_ext));
  const size_t lds = stage_bytes(a.group_rows, a.k);
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    auto kern = grouped_gemv_kernel<FMT, NB>;
    err = ensure_lds(kern, lds);
    if (err != hipSuccess) return;
    hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g, steps);
  });
  return err != hipSuccess ? err : hipGetLastError();
}
#endif  // DGPP_GEMV_IMPL

}  // namespace dgpp_amd
