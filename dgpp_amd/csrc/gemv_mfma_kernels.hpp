// Kernels of the matrix-core GEMV form (gemv_mfma.hpp): dense projection and grouped segments
// (row-wide tile loads, a block-shared activation stage), decode slots (one K part per wavefront).
// Included by gemv_kernels.hpp after the argument structs.
#pragma once

#include "gemv_mfma.hpp"

namespace dgpp_amd {

constexpr int kStageUnits = 1024;   // 16-byte units of one block-shared activation stage (16 KB)
constexpr int kMfmaNB = 4;          // lane loads in flight per row group and pass

// 64 weight rows (one row group per wavefront) against mt <= 16 activation rows, parts [p_lo, p_hi) of K.
// K is walked in batches of up to kTileBatch tiles (a tile = four steps of a row group, gemv_mfma.hpp):
// a wavefront puts all of a batch's weight loads in flight, the block then fetches the batch's
// activations into the LDS stage as [8-element block][row], and the tiles pass one after the other through
// the wavefront's own LDS region into the matrix core. Nothing of a wavefront is in flight while it
// computes; the other blocks of the CU cover that, so the kernel is kept small in registers and LDS
// (several blocks per CU) rather than pipelined inside the wavefront. `sum` receives the parts' sums added
// in ascending order. `act_rows`, when given, names the activation row of each of the mt rows (a gather
// folded into the stage load). LDS: the stage, then one tile region per wavefront. Every thread of the
// block must call.
// Activation rows that arrive already quantized to NVFP4 (the W4A4 form): e2m1 codes [rows, k / 2], one e4m3 scale per
// 16 elements [rows, scale_stride]; the row's fp32 global is applied by the caller's epilogue. A row's eight-element
// block decodes to eight FP16 values exactly (e2m1 x e4m3 needs six significant bits and stays inside [2^-10, 2688]),
// and so do the weights in this form: the matrix core multiplies the same numbers a block-scaled FP4 x FP4
// instruction would, with FP16 operands.
struct A4Src {
  const uint8_t* scales = nullptr;
  size_t scale_stride = 0;
  int row_base = 0;   // row of activation 0 when no row list is given
};
__device__ __forceinline__ uint4 load_act_block_nvfp4(const uint8_t* __restrict__ codes_row, const uint8_t* __restrict__ scale_row,
                                                      int k0, int k) {
  if (k0 >= k) return make_uint4(0u, 0u, 0u, 0u);
  const uint32_t codes = *reinterpret_cast<const uint32_t*>(codes_row + (k0 >> 1));
  float e;
  f16x2_t m;
  split_scale_f16(__builtin_amdgcn_cvt_f32_fp8(static_cast<uint32_t>(scale_row[k0 >> 4]), 0), e, m);
  const f16x2_t v0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, e, 0) * m;
  const f16x2_t v1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, e, 1) * m;
  const f16x2_t v2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, e, 2) * m;
  const f16x2_t v3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, e, 3) * m;
  return make_uint4(__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1), __builtin_bit_cast(uint32_t, v2),
                    __builtin_bit_cast(uint32_t, v3));
}

constexpr int kTileBatch = 2;   // 8 KB in flight per wavefront; more tiles cost registers, and blocks per CU count for more
constexpr int kBlockMfmaLdsUnits = kStageUnits + kWavesPerBlock * kTileUnits;

// A4: `act` holds NVFP4 codes (act_stride in BYTES) described by `a4`; the rows are then named by act_rows or start at
// a4.row_base.
template <int FMT, int NB, bool NT, bool SW = false, bool A4 = false>
__device__ __forceinline__ void block_rows_mfma(const MatRef& mat, const uint16_t* __restrict__ act, size_t act_stride,
                                                const int32_t* __restrict__ act_rows, int mt, int n, int k, int row0,
                                                const MGeom& g, int p_lo, int p_hi, uint4* __restrict__ lds,
                                                f32x4_t& sum, const uint16_t* __restrict__ act_up = nullptr,
                                                float limit = 0.f, const A4Src a4 = A4Src()) {
  static_assert(NB == 4, "a tile is four steps");
  constexpr int kSub = MTraits<FMT>::kSub;
  constexpr int kStepBlocks = MTraits<FMT>::kStepBlocks;
  constexpr int kStepElems = MTraits<FMT>::kStepElems;
  constexpr int kStageRegs = kStageUnits / kBlockThreads;
  const int chunks = k / MTraits<FMT>::kLoadElems;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const WideLane wl = wide_lane<FMT>(mat, row0, n, k);
  const ScaleLane sl = scale_lane<FMT>(mat, row0, n, k);
  uint4* region = lds + kStageUnits + wave * kTileUnits;
  const int cc = min(lane & 15, mt - 1);
  const bool aligned = (((reinterpret_cast<uintptr_t>(act) | reinterpret_cast<uintptr_t>(act_up)) & 15u) == 0) &&
                       ((act_stride & 7u) == 0);
  const int cpp = g.part_steps / NB;   // tiles per part: part_steps is a multiple of four
  const int batch = max(1, min(kTileBatch, kStageUnits / (mt * kStepBlocks * NB)));
  const int t_hi = p_hi * cpp;
  // this thread's pieces of a batch's activations: 8-element block kb of row c for each of its units
  int unit_kb[kStageRegs];
  size_t unit_row[kStageRegs];   // element offset of the unit's activation row
#pragma unroll
  for (int i = 0; i < kStageRegs; ++i) {
    const int idx = threadIdx.x + i * kBlockThreads;
    const int kb = idx / mt, c = idx - kb * mt;
    unit_kb[i] = kb;
    if constexpr (A4)   // the row itself: codes and scales have different strides
      unit_row[i] = act_rows ? static_cast<size_t>(act_rows[c]) : static_cast<size_t>(a4.row_base + c);
    else
      unit_row[i] = (act_rows ? static_cast<size_t>(act_rows[c]) : static_cast<size_t>(c)) * act_stride;
  }
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = p_lo * cpp; t0 < t_hi; t0 += batch) {
    const int tiles = min(batch, t_hi - t0);
    const int units = tiles * NB * kStepBlocks * mt;
    const int k_base = t0 * NB * kStepElems;
    uint4 pre[kStageRegs];
    auto ask_activations = [&]() {
#pragma unroll
      for (int i = 0; i < kStageRegs; ++i) {
        pre[i] = make_uint4(0u, 0u, 0u, 0u);
        if (threadIdx.x + i * kBlockThreads < units) {
          if constexpr (A4)
            pre[i] = load_act_block_nvfp4(reinterpret_cast<const uint8_t*>(act) + unit_row[i] * act_stride,
                                          a4.scales + unit_row[i] * a4.scale_stride, k_base + unit_kb[i] * 8, k);
          else
            pre[i] = load_act_block(act + unit_row[i], k_base + unit_kb[i] * 8, k, aligned);
          if constexpr (SW)   // the activation is SwiGLU(act, act_up), computed on its way into the stage
            pre[i] = swiglu_bf16x8(pre[i], load_act_block(act_up + unit_row[i], k_base + unit_kb[i] * 8, k, aligned), limit);
        }
      }
    };
    // NVFP4 activation rows are asked for BEFORE the weight tiles: loads return in order, so their decode and the
    // stage's barriers run while the weights are still on their way (measured: the W4A4 chain 1050 -> 1000 us; for BF16
    // rows, which need no decode, the order made no difference or cost a little, so they keep theirs).
    if constexpr (A4) ask_activations();
    uint4 tile[kTileBatch][4];
    uint32_t sc[kTileBatch][4];
    int valid[kTileBatch];
#pragma unroll
    for (int d = 0; d < kTileBatch; ++d) {
      const int step0 = (t0 + d) * NB;
      valid[d] = d < tiles ? max(0, min(NB, g.steps - step0)) : 0;
      issue_tile<NT>(wl, valid[d] > 0 ? step0 : g.steps, tile[d]);   // nothing to read: zeros, no loads
#pragma unroll
      for (int i = 0; i < 4; ++i) sc[d][i] = load_scale<FMT>(sl, i < valid[d] ? step0 + i : g.steps, chunks, mat.cs);
    }
    if constexpr (!A4) ask_activations();
    __syncthreads();   // the stage's readers of the batch before are through
#pragma unroll
    for (int i = 0; i < kStageRegs; ++i)
      if (threadIdx.x + i * kBlockThreads < units) lds[threadIdx.x + i * kBlockThreads] = pre[i];
    __syncthreads();
#pragma unroll
    for (int d = 0; d < kTileBatch; ++d) {
      if (d < tiles) {
        commit_tile(region, tile[d]);   // the region's earlier reads were issued before: LDS keeps a wavefront's order
        mfma_tile<FMT, A4>(region, sc[d], lds + (d * NB * kStepBlocks + (lane >> 4) * kSub) * mt + cc, mt, valid[d], acc);
        if ((t0 + d + 1) % cpp == 0) {   // a part ends: it joins the running sum, ((p0 + p1) + p2) + p3
          sum = (t0 + d + 1 == (p_lo + 1) * cpp) ? acc : sum + acc;
          acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
      }
    }
  }
}

// Stores a folded tile: lane (c = lane % 16, q = lane / 16) holds weight rows row0 + 4q .. + 3 of
// activation row c.
template <int FMT>
__device__ __forceinline__ void store_tile(const f32x4_t& v, float divisor, void* out, int out_f32, size_t out_row,
                                           int row0, int n, bool live) {
  if (!live) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int r = row0 + (lane >> 4) * 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (r + i < n) {
      const float x = finish_dot<FMT>(v[i], divisor);
      if (out_f32)
        static_cast<float*>(out)[out_row + r + i] = x;
      else
        static_cast<uint16_t*>(out)[out_row + r + i] = f32_to_bf16(x);
    }
  }
}

// `partials` null: all parts in one block, folded and stored. Otherwise blockIdx.z names the ONE part
// this block computes and its raw sums go to partials[part][row of out][n] (fp32); fold_parts_kernel
// then adds the parts in the same ascending order — the split form's bits are the unsplit form's.
// A4 (NVFP4 weights, unsplit only): NVFP4 activation rows, the grouped W4A4 kernel's walk and epilogue over rows c0...
template <int FMT, int NB, bool NT, bool SW, bool A4 = false>
__global__ __launch_bounds__(kBlockThreads, 2) void mfma_dense_kernel(DenseArgs a, MGeom g, float* partials) {
  extern __shared__ uint4 lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int row0 = (static_cast<int>(blockIdx.x) * kWavesPerBlock + wave) * kGroupRows;
  const int c0 = static_cast<int>(blockIdx.y) * kTileCols;
  const int mt = min(kTileCols, a.m - c0);
  const int c = lane & 15;
  f32x4_t sum;
  if constexpr (A4) {
    A4Src src;
    src.scales = a.a4_scales;
    src.scale_stride = a.a4_scale_stride;
    src.row_base = c0;
    block_rows_mfma<FMT, NB, NT, false, true>(a.mat, a.act, a.act_stride, nullptr, mt, a.n, a.k, row0, g, 0, g.parts, lds, sum,
                                              nullptr, 0.f, src);
    if (c < mt) {
      const float mul = a.a4_gs[c0 + c] * (1.0f / load_divisor<FMT>(a.global));
      const f32x4_t scaled = {sum[0] * mul, sum[1] * mul, sum[2] * mul, sum[3] * mul};
      store_tile<kFmtMxfp4>(scaled, 1.0f, a.out, a.out_f32, static_cast<size_t>(c0 + c) * a.out_stride, row0, a.n, true);
    }
    return;
  }
  if (partials == nullptr) {
    block_rows_mfma<FMT, NB, NT, SW>(a.mat, a.act + static_cast<size_t>(c0) * a.act_stride, a.act_stride, nullptr, mt, a.n,
                                 a.k, row0, g, 0, g.parts, lds, sum,
                                 SW ? a.act_up + static_cast<size_t>(c0) * a.act_stride : nullptr, a.limit);
    store_tile<FMT>(sum, load_divisor<FMT>(a.global), a.out, a.out_f32, static_cast<size_t>(c0 + c) * a.out_stride, row0,
                    a.n, c < mt);
    return;
  }
  const int part = static_cast<int>(blockIdx.z);
  block_rows_mfma<FMT, NB, NT, SW>(a.mat, a.act + static_cast<size_t>(c0) * a.act_stride, a.act_stride, nullptr, mt, a.n, a.k,
                               row0, g, part, part + 1, lds, sum,
                               SW ? a.act_up + static_cast<size_t>(c0) * a.act_stride : nullptr, a.limit);
  store_tile<kFmtMxfp4>(sum, 1.0f, partials, 1, (static_cast<size_t>(part) * a.m + c0 + c) * a.n, row0, a.n, c < mt);
}

// ---- K parts side by side inside one block ---------------------------------------------------------------------
// A dense launch whose row tiles barely fill the chip leaves one wavefront per SIMD walking all of K on its own.
// Here a block is sixteen wavefronts: TEAM t (four of them, one per row group) walks part t of K, so the four parts
// of a row group run side by side and the block folds them in LDS in the unsplit form's order, ((p0 + p1) + p2) + p3:
// the same bits, no workspace, no second launch. A team shares its own activation stage; the barriers are
// block-wide, which is sound because every part is walked as the same number of tiles (a trailing part's missing
// steps are zero loads).
// RG row groups per block (four, or two with half the stage for up to eight activation rows: two such blocks share
// a CU, which evens out a grid that just exceeds one round of the larger blocks).
template <int RG>
struct TeamShape {
  static constexpr int kTeamThreads = RG * kWave;                     // the wavefronts that share one part of K
  static constexpr int kThreads = kMaxParts * kTeamThreads;
  static constexpr int kStage = kStageUnits * RG / kWavesPerBlock;    // 16-byte units of one team's activation stage
  static constexpr int kLdsUnits = kMaxParts * kStage + (kThreads / kWave) * kTileUnits;
};

template <int FMT, int NB, bool NT, int RG>
__device__ __forceinline__ void team_rows_mfma(const MatRef& mat, const uint16_t* __restrict__ act, size_t act_stride, int mt,
                                               int n, int k, int row0, const MGeom& g, int team, uint4* __restrict__ lds,
                                               f32x4_t& sum) {
  static_assert(NB == 4, "a tile is four steps");
  using S = TeamShape<RG>;
  constexpr int kSub = MTraits<FMT>::kSub;
  constexpr int kStepBlocks = MTraits<FMT>::kStepBlocks;
  constexpr int kStepElems = MTraits<FMT>::kStepElems;
  constexpr int kStageRegs = S::kStage / S::kTeamThreads;
  const int chunks = k / MTraits<FMT>::kLoadElems;
  const int lane = threadIdx.x & (kWave - 1), tid = threadIdx.x % S::kTeamThreads;
  const WideLane wl = wide_lane<FMT>(mat, row0, n, k);
  const ScaleLane sl = scale_lane<FMT>(mat, row0, n, k);
  uint4* stage = lds + team * S::kStage;
  uint4* region = lds + kMaxParts * S::kStage + (threadIdx.x >> 6) * kTileUnits;
  const int cc = min(lane & 15, mt - 1);
  const bool aligned = ((reinterpret_cast<uintptr_t>(act) & 15u) == 0) && ((act_stride & 7u) == 0);
  const int cpp = g.part_steps / NB;
  const int batch = max(1, min(kTileBatch, S::kStage / (mt * kStepBlocks * NB)));
  const int t_lo = team * cpp, t_hi = t_lo + cpp;
  int unit_kb[kStageRegs];
  size_t unit_row[kStageRegs];
#pragma unroll
  for (int i = 0; i < kStageRegs; ++i) {
    const int idx = tid + i * S::kTeamThreads;
    const int kb = idx / mt, c = idx - kb * mt;
    unit_kb[i] = kb;
    unit_row[i] = static_cast<size_t>(c) * act_stride;
  }
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = t_lo; t0 < t_hi; t0 += batch) {
    const int tiles = min(batch, t_hi - t0);
    uint4 tile[kTileBatch][4];
    uint32_t sc[kTileBatch][4];
    int valid[kTileBatch];
#pragma unroll
    for (int d = 0; d < kTileBatch; ++d) {
      const int step0 = (t0 + d) * NB;
      valid[d] = d < tiles ? max(0, min(NB, g.steps - step0)) : 0;
      issue_tile<NT>(wl, valid[d] > 0 ? step0 : g.steps, tile[d]);
#pragma unroll
      for (int i = 0; i < 4; ++i) sc[d][i] = load_scale<FMT>(sl, i < valid[d] ? step0 + i : g.steps, chunks, mat.cs);
    }
    const int units = tiles * NB * kStepBlocks * mt;
    const int k_base = t0 * NB * kStepElems;
    uint4 pre[kStageRegs];
#pragma unroll
    for (int i = 0; i < kStageRegs; ++i) {
      pre[i] = make_uint4(0u, 0u, 0u, 0u);
      if (tid + i * S::kTeamThreads < units) pre[i] = load_act_block(act + unit_row[i], k_base + unit_kb[i] * 8, k, aligned);
    }
    __syncthreads();   // every team's readers of the batch before are through
#pragma unroll
    for (int i = 0; i < kStageRegs; ++i)
      if (tid + i * S::kTeamThreads < units) stage[tid + i * S::kTeamThreads] = pre[i];
    __syncthreads();
#pragma unroll
    for (int d = 0; d < kTileBatch; ++d) {
      if (d < tiles) {
        commit_tile(region, tile[d]);
        mfma_tile<FMT>(region, sc[d], stage + (d * NB * kStepBlocks + (lane >> 4) * kSub) * mt + cc, mt, valid[d], acc);
      }
    }
  }
  sum = acc;
}

template <int FMT, int NB, bool NT, int RG>
__global__ __launch_bounds__(TeamShape<RG>::kThreads) void mfma_dense_teams_kernel(DenseArgs a, MGeom g) {
  extern __shared__ uint4 lds[];
  using S = TeamShape<RG>;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int team = wave / RG, rg = wave % RG;
  const int row0 = (static_cast<int>(blockIdx.x) * RG + rg) * kGroupRows;
  const int c0 = static_cast<int>(blockIdx.y) * kTileCols;
  const int mt = min(kTileCols, a.m - c0);
  f32x4_t sum;
  team_rows_mfma<FMT, NB, NT, RG>(a.mat, a.act + static_cast<size_t>(c0) * a.act_stride, a.act_stride, mt, a.n, a.k, row0, g, team,
                                  lds, sum);
  // every wavefront parks its part's sums in its own tile region (its last operand reads were issued before: LDS
  // keeps a wavefront's order); team 0 folds the four parts of its row groups in ascending order and stores
  uint4* regions = lds + kMaxParts * S::kStage;
  regions[wave * kTileUnits + lane] = __builtin_bit_cast(uint4, sum);
  __syncthreads();
  if (team != 0) return;
  f32x4_t s = sum;
  s = s + __builtin_bit_cast(f32x4_t, regions[(RG + rg) * kTileUnits + lane]);
  s = (s + __builtin_bit_cast(f32x4_t, regions[(2 * RG + rg) * kTileUnits + lane])) +
      __builtin_bit_cast(f32x4_t, regions[(3 * RG + rg) * kTileUnits + lane]);
  const int c = lane & 15;
  store_tile<FMT>(s, load_divisor<FMT>(a.global), a.out, a.out_f32, static_cast<size_t>(c0 + c) * a.out_stride, row0, a.n, c < mt);
}

// Two dense problems of the same k and m in ONE launch (reference: launch_mma_gemv_fp8_bf16_pair,
// src/kernels/mma_gemv.cu:935-961 - two dependent-free projections sharing one ramp and drain): the first tiles0 row
// tiles of the grid belong to problem 0, the rest to problem 1; each block then does what mfma_dense_kernel does for
// its problem, so every row's chain is its single launch's. Split form: partials of problem 1 follow problem 0's.
template <int FMT, int NB, bool NT>
__global__ __launch_bounds__(kBlockThreads, 2) void mfma_dense_pair_kernel(DenseArgs a0, DenseArgs a1, int tiles0, MGeom g,
                                                                           float* partials) {
  extern __shared__ uint4 lds[];
  const bool second = static_cast<int>(blockIdx.x) >= tiles0;
  const DenseArgs& a = second ? a1 : a0;
  const int bx = static_cast<int>(blockIdx.x) - (second ? tiles0 : 0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int row0 = (bx * kWavesPerBlock + wave) * kGroupRows;
  const int c0 = static_cast<int>(blockIdx.y) * kTileCols;
  const int mt = min(kTileCols, a.m - c0);
  const int c = lane & 15;
  f32x4_t sum;
  if (partials == nullptr) {
    block_rows_mfma<FMT, NB, NT>(a.mat, a.act + static_cast<size_t>(c0) * a.act_stride, a.act_stride, nullptr, mt, a.n, a.k, row0,
                                 g, 0, g.parts, lds, sum);
    store_tile<FMT>(sum, load_divisor<FMT>(a.global), a.out, a.out_f32, static_cast<size_t>(c0 + c) * a.out_stride, row0, a.n,
                    c < mt);
    return;
  }
  const int part = static_cast<int>(blockIdx.z);
  block_rows_mfma<FMT, NB, NT>(a.mat, a.act + static_cast<size_t>(c0) * a.act_stride, a.act_stride, nullptr, mt, a.n, a.k, row0, g,
                               part, part + 1, lds, sum);
  float* mine = partials + (second ? static_cast<size_t>(g.parts) * a0.m * a0.n : 0);
  store_tile<kFmtMxfp4>(sum, 1.0f, mine, 1, (static_cast<size_t>(part) * a.m + c0 + c) * a.n, row0, a.n, c < mt);
}

// out[r][j] = finish(((p0 + p1) + p2) + p3) over partials[part][r][j].
template <int FMT>
__global__ void fold_parts_kernel(const float* __restrict__ partials, int parts, int m, int n, const float* global,
                                  void* out, int out_f32, size_t out_stride) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<int64_t>(m) * n) return;
  const int r = static_cast<int>(i / n), j = static_cast<int>(i - static_cast<int64_t>(r) * n);
  const size_t plane = static_cast<size_t>(m) * n;
  float s = partials[i];
  if (parts >= 2) s = s + partials[plane + i];
  if (parts >= 4) s = (s + partials[2 * plane + i]) + partials[3 * plane + i];
  const float x = finish_dot<FMT>(s, load_divisor<FMT>(global));
  const size_t at = static_cast<size_t>(r) * out_stride + j;
  if (out_f32)
    static_cast<float*>(out)[at] = x;
  else
    static_cast<uint16_t*>(out)[at] = f32_to_bf16(x);
}

// GU: the block computes its rows of the segment's gate AND up matrices (two walks over K, the same
// activations) and stores SwiGLU(bf16(gate), bf16(up)) — the bits of two launches and the elementwise kernel.
// GUW (with GU): the block's wavefronts split into gate walkers and up walkers (32 rows of each per block, grid.x twice
// as long) instead of every wavefront walking both matrices in turn: the same bits, taken for small grids.
// A4 (NVFP4 experts only, GU false): the activations are NVFP4 rows (a.act the codes, a.act_stride bytes per row,
// a.a4_scales / a.a4_gs); out = acc * (gs[row] * (1 / global)), the reference's epilogue (src/kernels/moe_w4a4.cu:424).
template <int FMT, int NB, bool NT, bool GU, bool A4 = false, bool GUW = false>
__global__ __launch_bounds__(kBlockThreads, 2) void mfma_grouped_kernel(GroupedArgs a, MGeom g) {
  extern __shared__ uint4 lds[];
  const DgppMoeSegment seg = a.segs[blockIdx.y];
  const int z0 = static_cast<int>(blockIdx.z) * a.rows_per_block;
  if (z0 >= seg.rows) return;
  const int z1 = min(seg.rows, z0 + a.rows_per_block);
  const float *gp = nullptr, *gp2 = nullptr;
  const MatRef mat = mat_of_view<FMT>(a.views[seg.expert * 3 + (GU ? 0 : a.which)], &gp);
  const float divisor = load_divisor<FMT>(gp);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int row0 = (static_cast<int>(blockIdx.x) * kWavesPerBlock + wave) * kGroupRows;
  const int c = lane & 15;
  for (int c0 = z0; c0 < z1; c0 += kTileCols) {
    const int mt = min(kTileCols, z1 - c0);
    f32x4_t sum;
    const size_t first = static_cast<size_t>(seg.row0 + c0);
    const uint16_t* act = a.act_rows ? a.act : a.act + first * a.act_stride;
    const int32_t* rows = a.act_rows ? a.act_rows + first : nullptr;
    if constexpr (GU && GUW) {
      // Two wavefronts walk gate rows, the other two the SAME rows of up (a block covers 32 rows of each): every
      // wavefront makes one walk - the one-matrix kernel's register budget, a wavefront more per SIMD than two walks
      // in turn cost - and the block's one activation stage serves both matrices. The up sums meet the gate sums in LDS.
      const int which = wave >> 1;
      const int row0g = (static_cast<int>(blockIdx.x) * 2 + (wave & 1)) * kGroupRows;
      const MatRef mw = mat_of_view<FMT>(a.views[seg.expert * 3 + which], &gp2);
      f32x4_t t;
      block_rows_mfma<FMT, NB, NT>(mw, act, a.act_stride, rows, mt, a.n, a.k, row0g, g, 0, g.parts, lds, t);
      // an up wavefront parks its sums in its own tile region (its last operand reads were issued before: LDS keeps a
      // wavefront's order); the gate wavefront of the same rows takes them after the barrier
      uint4* regions = lds + kStageUnits;
      if (which == 1) regions[wave * kTileUnits + lane] = __builtin_bit_cast(uint4, t);
      __syncthreads();
      if (which == 0) {
        const f32x4_t sum_up = __builtin_bit_cast(f32x4_t, regions[(wave + 2) * kTileUnits + lane]);
        const float *gp_up = nullptr;
        (void)mat_of_view<FMT>(a.views[seg.expert * 3 + 1], &gp_up);
        const float divisor_up = load_divisor<FMT>(gp_up);
        sum = t;
        if (a.gate_up == 2) {
          store_tile<FMT>(sum, divisor, a.out, 0, (first + c) * a.out_stride, row0g, a.n, c < mt);
          store_tile<FMT>(sum_up, divisor_up, a.out_up, 0, (first + c) * a.out_stride, row0g, a.n, c < mt);
        } else if (c < mt) {
          uint16_t* out = static_cast<uint16_t*>(a.out) + (first + c) * a.out_stride;
          const int r = row0g + (lane >> 4) * 4;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (r + i < a.n)
              out[r + i] = swiglu_bf16(finish_dot<FMT>(sum[i], divisor), finish_dot<FMT>(sum_up[i], divisor_up), a.limit);
        }
      }
    } else if constexpr (GU) {
      // one compiled walk, run for the gate matrix and again for the up matrix (kept a loop: register budget)
      f32x4_t sum_up = {0.f, 0.f, 0.f, 0.f};
      float divisor_up = 1.f;
#pragma unroll 1
      for (int w = 0; w < 2; ++w) {
        const MatRef mw = mat_of_view<FMT>(a.views[seg.expert * 3 + w], &gp2);
        f32x4_t t;
        block_rows_mfma<FMT, NB, NT>(mw, act, a.act_stride, rows, mt, a.n, a.k, row0, g, 0, g.parts, lds, t);
        const float dw = load_divisor<FMT>(gp2);
        if (w == 0) {
          sum = t;
        } else {
          sum_up = t;
          divisor_up = dw;
        }
      }
      if (a.gate_up == 2) {
        store_tile<FMT>(sum, divisor, a.out, 0, (first + c) * a.out_stride, row0, a.n, c < mt);
        store_tile<FMT>(sum_up, divisor_up, a.out_up, 0, (first + c) * a.out_stride, row0, a.n, c < mt);
      } else if (c < mt) {
        uint16_t* out = static_cast<uint16_t*>(a.out) + (first + c) * a.out_stride;
        const int r = row0 + (lane >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (r + i < a.n)
            out[r + i] = swiglu_bf16(finish_dot<FMT>(sum[i], divisor), finish_dot<FMT>(sum_up[i], divisor_up), a.limit);
      }
    } else if constexpr (A4) {
      A4Src src;
      src.scales = a.a4_scales;
      src.scale_stride = a.a4_scale_stride;
      src.row_base = static_cast<int>(first);
      block_rows_mfma<FMT, NB, NT, false, true>(mat, a.act, a.act_stride, rows, mt, a.n, a.k, row0, g, 0, g.parts, lds, sum,
                                                nullptr, 0.f, src);
      if (c < mt) {
        const size_t arow = rows ? static_cast<size_t>(rows[c]) : first + c;
        const float mul = a.a4_gs[arow] * (1.0f / divisor);
        const f32x4_t scaled = {sum[0] * mul, sum[1] * mul, sum[2] * mul, sum[3] * mul};
        store_tile<kFmtMxfp4>(scaled, 1.0f, a.out, a.out_f32, (first + c) * a.out_stride, row0, a.n, true);
      }
    } else {
      block_rows_mfma<FMT, NB, NT>(mat, act, a.act_stride, rows, mt, a.n, a.k, row0, g, 0, g.parts, lds, sum);
      store_tile<FMT>(sum, divisor, a.out, a.out_f32, (first + c) * a.out_stride, row0, a.n, c < mt);
    }
  }
}

// ---- decode slots: one K part per wavefront ----------------------------------------------------------
// A block's four wavefronts are 4 / parts row groups times `parts` K parts. Each wavefront stages
// ITS part of the run's activation rows ([block][row], m <= MAXM rows) in its own LDS region, streams
// its 16 rows over that part, and the part sums meet in LDS, added in ascending part order by the
// part-0 wavefront (the block form's order).
template <int FMT>
__host__ __device__ inline int slot_wave_units(int maxm, const MGeom& g) {
  return maxm * g.part_steps * MTraits<FMT>::kStepBlocks;
}
constexpr int kSlotRedUnits = kWavesPerBlock * 2 * kWave;   // f32x4 per lane, two tiles per wavefront

template <int MAXM>
__device__ __forceinline__ int pick_slot(const int (&v)[MAXM], int c) {
  int s = v[0];
#pragma unroll
  for (int r = 1; r < MAXM; ++r) s = c == r ? v[r] : s;
  return s;
}

// Stages rows x + idx[0 .. m-1] * x_stride (k bf16 values each) of this wavefront's K part.
template <int FMT, int MAXM>
__device__ __forceinline__ void stage_wave_part(const uint16_t* __restrict__ x, size_t x_stride, const int (&idx)[MAXM],
                                                int m, int k, int part, const MGeom& g, uint4* __restrict__ stage) {
  const int lane = threadIdx.x & (kWave - 1);
  const int k_base = part * g.part_steps * MTraits<FMT>::kStepElems;
  const int units = g.part_steps * MTraits<FMT>::kStepBlocks * m;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) && ((x_stride & 7u) == 0);
  for (int u = lane; u < units; u += kWave) {
    const int kb = u / m, r = u - kb * m;
    const uint16_t* row = x + static_cast<size_t>(pick_slot<MAXM>(idx, r)) * x_stride;
    stage[u] = load_act_block(row, k_base + kb * 8, k, aligned);
  }
}

template <int FMT, int NB, int MAXM>
__global__ __launch_bounds__(kBlockThreads, 2) void slot_gate_up_mfma_kernel(SlotArgs a, MGeom g) {
  extern __shared__ uint4 lds[];
  SlotRun<MAXM> run;
  if (!resolve_run<MAXM>(a, run)) return;
  const int gpb = kWavesPerBlock / g.parts;   // row groups per block
  if (static_cast<int>(blockIdx.x) * gpb * kGroupRows >= a.n) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int grp = wave / g.parts, part = wave - grp * g.parts;
  const int row0 = (static_cast<int>(blockIdx.x) * gpb + grp) * kGroupRows;
  MatRef mg, mu;
  const float *gg = nullptr, *gu = nullptr;
  if (run.view_base >= 0) {
    mg = mat_of_view<FMT>(a.views[run.view_base + 0], &gg);
    mu = mat_of_view<FMT>(a.views[run.view_base + 1], &gu);
  } else {
    mg = a.sh[0];
    mu = a.sh[1];
  }
  const int m = run.m;
  const int wave_units = slot_wave_units<FMT>(MAXM, g);
  uint4* stage = lds + wave * wave_units;
  f32x4_t* red = reinterpret_cast<f32x4_t*>(lds + kWavesPerBlock * wave_units);
  stage_wave_part<FMT, MAXM>(a.x, a.x_stride, run.token, m, a.k, part, g, stage);
  __syncthreads();
  constexpr int kSub = MTraits<FMT>::kSub;
  constexpr int kStepBlocks = MTraits<FMT>::kStepBlocks;
  const int chunks = a.k / MTraits<FMT>::kLoadElems;
  const auto lg = group_lane<FMT, true>(mg, row0, a.n, a.k);
  const auto lu = group_lane<FMT, true>(mu, row0, a.n, a.k);
  const int cc = min(lane & 15, m - 1);
  const uint4* lane_stage = stage + ((lane >> 4) * kSub) * m + cc;
  const int step0 = part * g.part_steps;
  const int nsteps = min(g.part_steps, g.steps - step0);
  f32x4_t ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
  for (int t = 0; t < nsteps; t += NB) {
    ChunkRegs rg[NB], ru[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int st = t + i < nsteps ? step0 + t + i : g.steps;
      load_step<FMT>(lg, st, chunks, mg.cs, rg[i]);
      load_step<FMT>(lu, st, chunks, mu.cs, ru[i]);
    }
    mfma_chunk_pair<FMT, NB>(lg, rg, ru, lane_stage + (t * kStepBlocks) * m, m, min(NB, nsteps - t), ag, au);
  }
  if (g.parts > 1) {
    if (part != 0) {
      red[(wave * 2 + 0) * kWave + lane] = ag;
      red[(wave * 2 + 1) * kWave + lane] = au;
    }
    __syncthreads();
    if (part != 0) return;
    ag = ag + red[((wave + 1) * 2 + 0) * kWave + lane];
    au = au + red[((wave + 1) * 2 + 1) * kWave + lane];
    if (g.parts == 4) {
      ag = (ag + red[((wave + 2) * 2 + 0) * kWave + lane]) + red[((wave + 3) * 2 + 0) * kWave + lane];
      au = (au + red[((wave + 2) * 2 + 1) * kWave + lane]) + red[((wave + 3) * 2 + 1) * kWave + lane];
    }
  }
  const int c = lane & 15;
  if (c >= m) return;
  const float dg = load_divisor<FMT>(gg), du = load_divisor<FMT>(gu);
  uint16_t* act_row = static_cast<uint16_t*>(a.out) + static_cast<size_t>(pick_slot<MAXM>(run.slot, c)) * a.out_stride;
  const int r = row0 + (lane >> 4) * 4;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (r + i < a.n) act_row[r + i] = swiglu_bf16(finish_dot<FMT>(ag[i], dg), finish_dot<FMT>(au[i], du), a.limit);
}

template <int FMT, int NB, int MAXM>
__global__ __launch_bounds__(kBlockThreads, 2) void slot_down_mfma_kernel(SlotArgs a, MGeom g) {
  extern __shared__ uint4 lds[];
  SlotRun<MAXM> run;
  if (!resolve_run<MAXM>(a, run)) return;
  const int gpb = kWavesPerBlock / g.parts;
  if (static_cast<int>(blockIdx.x) * gpb * kGroupRows >= a.n) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int grp = wave / g.parts, part = wave - grp * g.parts;
  const int row0 = (static_cast<int>(blockIdx.x) * gpb + grp) * kGroupRows;
  MatRef md;
  const float* gd = nullptr;
  if (run.view_base >= 0)
    md = mat_of_view<FMT>(a.views[run.view_base + 2], &gd);
  else
    md = a.sh[0];
  const int m = run.m;
  const int wave_units = slot_wave_units<FMT>(MAXM, g);
  uint4* stage = lds + wave * wave_units;
  f32x4_t* red = reinterpret_cast<f32x4_t*>(lds + kWavesPerBlock * wave_units);
  stage_wave_part<FMT, MAXM>(a.x, a.x_stride, run.slot, m, a.k, part, g, stage);
  __syncthreads();
  constexpr int kSub = MTraits<FMT>::kSub;
  constexpr int kStepBlocks = MTraits<FMT>::kStepBlocks;
  const int chunks = a.k / MTraits<FMT>::kLoadElems;
  const auto ld = group_lane<FMT, true>(md, row0, a.n, a.k);
  const int cc = min(lane & 15, m - 1);
  const uint4* lane_stage = stage + ((lane >> 4) * kSub) * m + cc;
  const int step0 = part * g.part_steps;
  const int nsteps = min(g.part_steps, g.steps - step0);
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int t = 0; t < nsteps; t += NB) {
    ChunkRegs regs[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) load_step<FMT>(ld, t + i < nsteps ? step0 + t + i : g.steps, chunks, md.cs, regs[i]);
    mfma_chunk<FMT, NB>(ld, regs, lane_stage + (t * kStepBlocks) * m, m, min(NB, nsteps - t), acc);
  }
  if (g.parts > 1) {
    if (part != 0) red[wave * kWave + lane] = acc;
    __syncthreads();
    if (part != 0) return;
    acc = acc + red[(wave + 1) * kWave + lane];
    if (g.parts == 4) acc = (acc + red[(wave + 2) * kWave + lane]) + red[(wave + 3) * kWave + lane];
  }
  const int c = lane & 15;
  store_tile<FMT>(acc, load_divisor<FMT>(gd), a.out, 1,
                  static_cast<size_t>(pick_slot<MAXM>(run.slot, c)) * a.out_stride, row0, a.n, c < m);
}

}  // namespace dgpp_amd
