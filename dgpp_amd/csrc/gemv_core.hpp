// The weight-streaming GEMV core for gfx950 (wave64), shared by the dense projection
// launchers, the MoE decode-slot kernels and the grouped (segment-major) kernels.
//
// Shape of the computation. A weight row is a string of 16-byte CHUNKS (16 FP8 codes or
// 32 FP4 codes). A row is covered by L = 2^l2 adjacent lanes (L <= 64); lane li of the row
// owns chunks li, li + L, li + 2L, ... (P of them), so one load instruction of a row group
// reads L consecutive chunks: fully coalesced 16-byte-per-lane global loads. A wavefront
// carries 64 / L rows per step. Each lane decodes its chunks in registers to packed bf16
// pairs (hardware FP4 / FP8 conversions of gfx950), multiplies them with the activation
// vector staged in LDS through v_dot2_f32_bf16 (fp32 accumulate), and the L partial sums of
// a row are folded by a fixed DPP / lane-permute butterfly. (row, activation-row) results
// therefore depend only on (format, k): never on how many activation rows share the launch,
// on the launcher, or on the grid — the property the slot / grouped / dense launchers'
// bitwise-twin tests pin.
//
// Value semantics (reference: src/kernels/fp8_gemv.cuh:64-66, src/kernels/fp4_gemv.cuh:20-27):
//   FP8 + F32 grid   w = bf16_rne(float(e4m3) * scale)               (the rounding is part of the value)
//   FP8 + E8M0 grid  w = e4m3 * 2^(b-127), b == 0 -> 2^-127          (exact in bf16; byte 255 gives NaN, the
//                    E8M0 encoding's meaning, where the reference's dequant bridge reads it as +inf)
//   NVFP4            w = e2m1 * e4m3(scale) exact; dot / global once  (we sum a 16-group unscaled,
//                    then fold the group scale in with one fma: same sum, fp32 rounding order only)
//   MXFP4            w = e2m1 * 2^(b-127) exact, b == 255 -> NaN
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "numerics.hpp"

namespace dgpp_amd {

enum : int { kFmtFp8F32 = 0, kFmtFp8E8M0 = 1, kFmtNvfp4 = 2, kFmtMxfp4 = 3 };

constexpr int kWave = 64;
constexpr int kBlockThreads = 256;
constexpr int kWavesPerBlock = kBlockThreads / kWave;
constexpr int kChunkBytes = 16;
constexpr int kMaxActRows = 8;                 // activation rows one launch carries
constexpr size_t kDefaultLdsBytes = 64 * 1024;  // dynamic LDS a block may take without opt-in
constexpr size_t kMaxLdsBytes = 160 * 1024;     // LDS of one gfx950 CU: the ceiling after opt-in

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;

template <int FMT>
struct FmtTraits {
  static constexpr bool kIsFp4 = FMT >= kFmtNvfp4;
  static constexpr int kElemsPerChunk = kIsFp4 ? 32 : 16;
  static constexpr int kPieces = kElemsPerChunk / 8;  // 16-byte activation vectors per chunk
};

// One weight matrix as the core reads it.
struct MatRef {
  const uint8_t* payload;   // [n, row_bytes]
  const void* scales;       // FP8: float or e8m0 grid; FP4: per-row scale bytes
  float divisor;            // NVFP4: the device global (dot divided by it); else unused
  int rs, cs;               // FP8 scale grid log2 block sizes
};

// Row geometry as a function of the chunk count of a row.
struct RowGeom {
  int l2;      // log2 lanes per row
  int P;       // chunks per lane
  int nb;      // chunks per pass (a divisor of P, <= 8): the loads in flight per lane per row
};
// Bench A/B switches (host side, process-wide; 0 = the default behaviour). Set through
// dgpp_tune_set; launchers read them when they pick a geometry or a kernel form.
enum : int { kTunePreferP = 0, kTuneSlotRun = 1, kTuneSlotSteps = 2, kTuneSplitStage = 3, kTuneCore = 5, kTuneSelectAlone = 7, kTuneXcdGroup = 8, kTuneRouterTile = 10, kTuneTeams = 11, kTuneChain = 12, kTuneChainDownSteps = 13, kTuneGateUpWalks = 14, kTuneCount = 15 };
int tune_get(int key);

__host__ __device__ inline RowGeom row_geom(int chunks, int prefer_p = 4) {
  RowGeom g;
  g.l2 = 0;
  while (g.l2 < 6 && (chunks % (2 << g.l2)) == 0) ++g.l2;
  g.P = chunks >> g.l2;
  // Prefer at least `prefer_p` chunks per lane over very wide row groups (a row group keeps at
  // least 128 contiguous bytes per load instruction: 8 lanes). Four measured a few percent faster
  // than two on the MoE shapes (more bytes in flight per lane).
  while (g.P < prefer_p && g.l2 > 3) {
    --g.l2;
    g.P *= 2;
  }
  g.nb = 1;
  for (int d = 8; d >= 1; --d)
    if (d != 7 && g.P % d == 0) {
      g.nb = d;
      break;
    }
  return g;
}

// ---- activation staging -----------------------------------------------------------------
// LDS layout: 16-byte vectors indexed [(r * kPieces + q) * chunks + c] for activation row r,
// chunk c, piece q (elements 8q .. 8q+7 of the chunk). Lanes of a row group read consecutive
// c for a fixed q: consecutive 16-byte vectors, bank-conflict free.
template <int FMT>
__device__ __forceinline__ void stage_activations(const uint16_t* __restrict__ x, size_t x_stride,
                                                  int rows, int k, uint4* __restrict__ lds) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
  const int chunks = k / FmtTraits<FMT>::kElemsPerChunk;
  const int vecs = k / 8;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) && ((x_stride & 7u) == 0);
  if (aligned) {
    for (int i = threadIdx.x; i < rows * vecs; i += blockDim.x) {
      const int r = i / vecs, v = i - r * vecs;
      const int c = v / kPieces, q = v - c * kPieces;
      lds[(r * kPieces + q) * chunks + c] =
          *reinterpret_cast<const uint4*>(x + static_cast<size_t>(r) * x_stride + static_cast<size_t>(v) * 8);
    }
  } else {
    uint16_t* l16 = reinterpret_cast<uint16_t*>(lds);
    for (int i = threadIdx.x; i < rows * k; i += blockDim.x) {
      const int r = i / k, e = i - r * k;
      const int v = e >> 3, c = v / kPieces, q = v - c * kPieces;
      l16[(static_cast<size_t>((r * kPieces + q) * chunks + c) << 3) + (e & 7)] =
          x[static_cast<size_t>(r) * x_stride + e];
    }
  }
}

// Vector v (8 bf16 values) of an activation row.
__device__ __forceinline__ uint4 load_vec8(const uint16_t* __restrict__ x, int v, bool aligned) {
  if (aligned) return *reinterpret_cast<const uint4*>(x + static_cast<size_t>(v) * 8);
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = static_cast<uint32_t>(x[v * 8 + 2 * i]) | (static_cast<uint32_t>(x[v * 8 + 2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// ---- lane butterflies ---------------------------------------------------------------------
template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xF, 0xF, true));
}
// Sum over the 2^l2 adjacent lanes of a row group; every lane of the group gets the sum.
// Fixed order: distances 1, 2 (quad permutes), 4, 8 (half-row / row mirrors: after the
// earlier steps every lane of a quad / octet already holds the same partial, so a mirror
// pairs the same partials as an xor would), then 16 and 32 by lane permutes.
__device__ __forceinline__ float group_sum(float v, int l2) {
  if (l2 >= 1) v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  if (l2 >= 2) v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  if (l2 >= 3) v += dpp_move<0x141>(v);  // row_half_mirror
  if (l2 >= 4) v += dpp_move<0x140>(v);  // row_mirror
  if (l2 >= 5) v += __shfl_xor(v, 16);
  if (l2 >= 6) v += __shfl_xor(v, 32);
  return v;
}

// ---- per-chunk arithmetic -------------------------------------------------------------------
__device__ __forceinline__ float dot2(bf16x2_t w, uint32_t xpair, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(w, __builtin_bit_cast(bf16x2_t, xpair), acc, false);
}
__device__ __forceinline__ bf16x2_t pack_bf16(float a, float b) {
  f32x2_t v = {a, b};
  return __builtin_convertvector(v, bf16x2_t);
}

// The raw bytes a lane holds for one chunk: 16 payload bytes and its scale word.
struct ChunkRegs {
  uint4 w;
  uint32_t s;  // FP8-F32: float bits; FP8-E8M0 / MXFP4: the byte; NVFP4: two e4m3 bytes
};

// Issues the loads of chunk index c of the row whose payload / scale rows are given.
// NT: the launch reads every weight once. Nontemporal loads then keep the stream from displacing the
// activations and the expert table in the caches (measured: the decode gate/up kernel 9 % faster); where
// weights are read again (several activation tiles, many slots per expert) the cached form wins. A compile
// time choice on purpose: a run-time branch between two otherwise identical loads gets merged into one
// plain load by the optimiser.
template <int FMT, bool NT>
__device__ __forceinline__ void load_chunk(const uint8_t* __restrict__ payload_row,
                                           const void* __restrict__ scale_row, int c, int cs,
                                           ChunkRegs& out) {
  // Weights live in global memory (never LDS or scratch): saying so lets the loads be global_load
  // instead of flat_load.
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
#define DGPP_AS1 __attribute__((address_space(1)))
  const DGPP_AS1 u32x4_t* src = (const DGPP_AS1 u32x4_t*)(uintptr_t)(payload_row + static_cast<size_t>(c) * kChunkBytes);
  const u32x4_t v = NT ? __builtin_nontemporal_load(src) : *src;
  out.w = make_uint4(v.x, v.y, v.z, v.w);
  if constexpr (FMT == kFmtFp8F32) {
    out.s = ((const DGPP_AS1 uint32_t*)(uintptr_t)scale_row)[((c * 16) >> cs)];
  } else if constexpr (FMT == kFmtFp8E8M0) {
    out.s = ((const DGPP_AS1 uint8_t*)(uintptr_t)scale_row)[((c * 16) >> cs)];
  } else if constexpr (FMT == kFmtNvfp4) {
    out.s = ((const DGPP_AS1 uint16_t*)(uintptr_t)scale_row)[c];
  } else {
    out.s = ((const DGPP_AS1 uint8_t*)(uintptr_t)scale_row)[c];
  }
#undef DGPP_AS1
}

// Where a chunk's activation vectors come from: LDS (any number of staged rows) ...
template <int FMT>
struct XLds {
  const uint4* base;  // LDS vector [piece 0][chunk c] of activation row 0
  int chunks;
  __device__ __forceinline__ uint4 get(int r, int q) const { return base[(r * FmtTraits<FMT>::kPieces + q) * chunks]; }
};
// ... or registers (one activation row, the lane's own chunk columns loaded once per wavefront).
template <int FMT>
struct XReg {
  const uint4* v;     // [kPieces] vectors of this chunk
  __device__ __forceinline__ uint4 get(int, int q) const { return v[q]; }
};

// ---- per-chunk arithmetic, split in decode and dot ------------------------------------------------
// A chunk decoded to packed bf16 pairs (element pairs in k order); NVFP4 keeps its two group scales
// aside because they are folded in once per 16-group, after the unscaled partial sum.
template <int FMT>
struct Decoded {
  bf16x2_t p[FmtTraits<FMT>::kElemsPerChunk / 2];
  float s0, s1;
};

template <int FMT>
__device__ __forceinline__ void decode_chunk(const ChunkRegs& ch, Decoded<FMT>& d) {
  const uint32_t w[4] = {ch.w.x, ch.w.y, ch.w.z, ch.w.w};
  if constexpr (FMT == kFmtMxfp4 || FMT == kFmtNvfp4) {
    // MXFP4: the scaled conversion takes the E8M0 byte as the exponent field of a float and is exact
    // for EVERY byte on gfx950 (0 -> 2^-127 with subnormal bf16 results, 255 -> NaN), checked over all
    // 256 x 16 (byte, code) pairs on the hardware.
    const float s = FMT == kFmtMxfp4 ? bits_f32(ch.s << 23) : 1.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      d.p[q * 4 + 0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 0);
      d.p[q * 4 + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 1);
      d.p[q * 4 + 2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 2);
      d.p[q * 4 + 3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 3);
    }
    if constexpr (FMT == kFmtNvfp4) {
      // The two e4m3 group scales (codes 0..15 and 16..31); NaN codes propagate.
      d.s0 = __builtin_amdgcn_cvt_f32_fp8(ch.s, 0);
      d.s1 = __builtin_amdgcn_cvt_f32_fp8(ch.s, 1);
    }
  } else if constexpr (FMT == kFmtFp8E8M0) {
    const float s = bits_f32(ch.s << 23);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      d.p[q * 2 + 0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[q], s, false);
      d.p[q * 2 + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[q], s, true);
    }
  } else {
    // float(e4m3) * scale in fp32, one RNE rounding to bf16: the rounding is part of the value.
    const float s = bits_f32(ch.s);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[q], false);
      const f32x2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[q], true);
      d.p[q * 2 + 0] = pack_bf16(lo.x * s, lo.y * s);
      d.p[q * 2 + 1] = pack_bf16(hi.x * s, hi.y * s);
    }
  }
}

// acc + dot(decoded chunk, the chunk's activation vectors x[0 .. kPieces)).
template <int FMT>
__device__ __forceinline__ float dot_chunk(const Decoded<FMT>& d, const uint4* x, float acc) {
  if constexpr (FMT == kFmtNvfp4) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float part = 0.f;
#pragma unroll
      for (int q = 2 * h; q < 2 * h + 2; ++q) {
        part = dot2(d.p[q * 4 + 0], x[q].x, part);
        part = dot2(d.p[q * 4 + 1], x[q].y, part);
        part = dot2(d.p[q * 4 + 2], x[q].z, part);
        part = dot2(d.p[q * 4 + 3], x[q].w, part);
      }
      acc = fmaf(part, h == 0 ? d.s0 : d.s1, acc);
    }
  } else {
#pragma unroll
    for (int q = 0; q < FmtTraits<FMT>::kPieces; ++q) {
      acc = dot2(d.p[q * 4 + 0], x[q].x, acc);
      acc = dot2(d.p[q * 4 + 1], x[q].y, acc);
      acc = dot2(d.p[q * 4 + 2], x[q].z, acc);
      acc = dot2(d.p[q * 4 + 3], x[q].w, acc);
    }
  }
  return acc;
}

// acc[r] += dot(chunk weights, activation row r's elements of the chunk) for r < m.
template <int FMT, int MAXR, class X>
__device__ __forceinline__ void consume_chunk(const ChunkRegs& ch, const X& xs, int m, float (&acc)[MAXR]) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
  Decoded<FMT> d;
  decode_chunk<FMT>(ch, d);
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < m) {
      uint4 xv[kPieces];
#pragma unroll
      for (int q = 0; q < kPieces; ++q) xv[q] = xs.get(r, q);
      acc[r] = dot_chunk<FMT>(d, xv, acc[r]);
    }
  }
  // Keep the scheduler from hoisting the next chunk's decode above this chunk's dots: that trades
  // a few cycles of overlap for dozens of live registers (and spills) per lane.
  __builtin_amdgcn_sched_barrier(0);
}

// ---- a wavefront's row step --------------------------------------------------------------------
// Per-lane addressing of one row step: which row this lane helps with and where its chunks start.
struct LaneRow {
  const uint8_t* payload_row;
  const void* scale_row;
  int row;       // absolute row (may be >= n: the lane then works on row n-1 and its result is dropped)
  int li;        // lane index inside the row group
};

// The row with the load policy (load_chunk's NT) as part of its type: functions that issue loads deduce it.
template <bool NT>
struct LaneRowT : LaneRow {
  static constexpr bool kNT = NT;
};

template <int FMT, bool NT = true>
__device__ __forceinline__ LaneRowT<NT> lane_row(const MatRef& mat, int row0, int n, int k, int l2) {
  const int lane = threadIdx.x & (kWave - 1);
  LaneRowT<NT> lr;
  lr.li = lane & ((1 << l2) - 1);
  lr.row = row0 + (lane >> l2);
  const int r = lr.row < n ? lr.row : n - 1;
  if constexpr (FMT == kFmtFp8F32 || FMT == kFmtFp8E8M0) {
    lr.payload_row = mat.payload + static_cast<size_t>(r) * k;
    const size_t scale_cols = (static_cast<size_t>(k) + (1u << mat.cs) - 1) >> mat.cs;
    const size_t esz = FMT == kFmtFp8F32 ? 4 : 1;
    lr.scale_row = reinterpret_cast<const uint8_t*>(mat.scales) + (static_cast<size_t>(r >> mat.rs) * scale_cols) * esz;
  } else {
    lr.payload_row = mat.payload + static_cast<size_t>(r) * (k / 2);
    lr.scale_row = reinterpret_cast<const uint8_t*>(mat.scales) +
                   static_cast<size_t>(r) * (k / (FMT == kFmtNvfp4 ? 16 : 32));
  }
  return lr;
}

// Loads one pass (NB chunks) of a row for this lane.
template <int FMT, int NB, class LR>
__device__ __forceinline__ void issue_pass(const LR& lr, int pass, int l2, int cs,
                                           ChunkRegs (&regs)[NB]) {
#pragma unroll
  for (int i = 0; i < NB; ++i)
    load_chunk<FMT, LR::kNT>(lr.payload_row, lr.scale_row, ((pass * NB + i) << l2) + lr.li, cs, regs[i]);
}

template <int FMT, int MAXR, int NB>
__device__ __forceinline__ void consume_pass(const ChunkRegs (&regs)[NB], const LaneRow& lr, int pass,
                                             int l2, const uint4* __restrict__ lds, int chunks, int m,
                                             float (&acc)[MAXR]) {
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int c = ((pass * NB + i) << l2) + lr.li;
    consume_chunk<FMT, MAXR>(regs[i], XLds<FMT>{lds + c, chunks}, m, acc);
  }
}

// Full dot products of this lane's row against m staged activation rows; after the call every
// lane of the row group holds the finished sums (the NVFP4 division is the caller's epilogue).
template <int FMT, int MAXR, int NB, class LR>
__device__ __forceinline__ void row_dots(const LR& lr, const RowGeom& g, int cs,
                                         const uint4* __restrict__ lds, int chunks, int m,
                                         float (&acc)[MAXR]) {
#pragma unroll
  for (int r = 0; r < MAXR; ++r) acc[r] = 0.f;
  const int passes = g.P / NB;
  for (int p = 0; p < passes; ++p) {
    ChunkRegs cur[NB];
    issue_pass<FMT, NB>(lr, p, g.l2, cs, cur);
    consume_pass<FMT, MAXR, NB>(cur, lr, p, g.l2, lds, chunks, m, acc);
  }
#pragma unroll
  for (int r = 0; r < MAXR; ++r)
    if (r < m) acc[r] = group_sum(acc[r], g.l2);
}

// row_dots with the first pass's loads already issued by the caller. Same chain.
template <int FMT, int MAXR, int NB, class LR>
__device__ __forceinline__ void row_dots_pre(const LR& lr, const RowGeom& g, int cs,
                                             const uint4* __restrict__ lds, int chunks, int m,
                                             const ChunkRegs (&first)[NB], float (&acc)[MAXR]) {
#pragma unroll
  for (int r = 0; r < MAXR; ++r) acc[r] = 0.f;
  consume_pass<FMT, MAXR, NB>(first, lr, 0, g.l2, lds, chunks, m, acc);
  const int passes = g.P / NB;
  for (int p = 1; p < passes; ++p) {
    ChunkRegs cur[NB];
    issue_pass<FMT, NB>(lr, p, g.l2, cs, cur);
    consume_pass<FMT, MAXR, NB>(cur, lr, p, g.l2, lds, chunks, m, acc);
  }
#pragma unroll
  for (int r = 0; r < MAXR; ++r)
    if (r < m) acc[r] = group_sum(acc[r], g.l2);
}

// Activation staging split in two so that weight loads can be issued in between: the activation loads
// go out first (memory returns a wavefront's loads in order, so waiting for them does not wait for the
// younger weight loads), are committed to LDS after the weights are on their way. One row of k <= 8 * XV
// * threads elements, 16-byte aligned; vector v goes to [(piece) * chunks + chunk] of `dst`.
template <int XV>
struct StageRegs {
  uint4 v[XV];
};
template <int FMT, int XV>
__device__ __forceinline__ void stage_issue(const uint16_t* __restrict__ x, int k, int tid, int threads, StageRegs<XV>& r) {
  const int vecs = k / 8;
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    const int v = tid + i * threads;
    r.v[i] = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(v < vecs ? v : 0) * 8);   // always defined
  }
}
template <int FMT, int XV>
__device__ __forceinline__ void stage_commit(const StageRegs<XV>& r, int k, int tid, int threads, uint4* __restrict__ dst) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
  const int chunks = k / FmtTraits<FMT>::kElemsPerChunk;
  const int vecs = k / 8;
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    const int v = tid + i * threads;
    if (v < vecs) {
      const int c = v / kPieces, q = v - c * kPieces;
      dst[q * chunks + c] = r.v[i];
    }
  }
}

// One activation row already in registers: acc + dot(chunk, x).
template <int FMT>
__device__ __forceinline__ float chunk_dot1(const ChunkRegs& ch, const uint4* xv, float acc) {
  Decoded<FMT> d;
  decode_chunk<FMT>(ch, d);
  acc = dot_chunk<FMT>(d, xv, acc);
  __builtin_amdgcn_sched_barrier(0);
  return acc;
}

// Two weight rows of the same geometry (a slot's gate and up rows) against the SAME m staged
// activation rows: both rows' loads are issued together and each chunk column's activation vectors
// are read from LDS once for the pair. Each (row, activation row) chain is row_dots' chain, bit for
// bit.
// One pass of a gate / up row pair against the m staged rows.
template <int FMT, int NB, int MAXM>
__device__ __forceinline__ void consume_pass_pair(const ChunkRegs (&ca)[NB], const ChunkRegs (&cb)[NB], int li, int p,
                                                  int l2, const uint4* __restrict__ lds, int chunks, int m,
                                                  float (&ra)[MAXM], float (&rb)[MAXM]) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int c = ((p * NB + i) << l2) + li;
    if constexpr (MAXM == 1) {
      uint4 xv[kPieces];
#pragma unroll
      for (int q = 0; q < kPieces; ++q) xv[q] = lds[q * chunks + c];
      ra[0] = chunk_dot1<FMT>(ca[i], xv, ra[0]);
      rb[0] = chunk_dot1<FMT>(cb[i], xv, rb[0]);
    } else {
      consume_chunk<FMT, MAXM>(ca[i], XLds<FMT>{lds + c, chunks}, m, ra);
      consume_chunk<FMT, MAXM>(cb[i], XLds<FMT>{lds + c, chunks}, m, rb);
    }
  }
}
template <int FMT, int NB, int MAXM, class LR>
__device__ __forceinline__ void row_dots_pair(const LR& la, const LR& lb, const RowGeom& g, int csa,
                                              int csb, const uint4* __restrict__ lds, int chunks, int m,
                                              float (&ra)[MAXM], float (&rb)[MAXM]) {
#pragma unroll
  for (int r = 0; r < MAXM; ++r) ra[r] = rb[r] = 0.f;
  const int passes = g.P / NB;
  for (int p = 0; p < passes; ++p) {
    ChunkRegs ca[NB], cb[NB];
    issue_pass<FMT, NB>(la, p, g.l2, csa, ca);
    issue_pass<FMT, NB>(lb, p, g.l2, csb, cb);
    consume_pass_pair<FMT, NB, MAXM>(ca, cb, la.li, p, g.l2, lds, chunks, m, ra, rb);
  }
#pragma unroll
  for (int r = 0; r < MAXM; ++r) {
    if (r < m) {
      ra[r] = group_sum(ra[r], g.l2);
      rb[r] = group_sum(rb[r], g.l2);
    }
  }
}
// The same with pass 0 of the two rows already issued by the caller (`fa`, `fb`). Same chain.
template <int FMT, int NB, int MAXM, class LR>
__device__ __forceinline__ void row_dots_pair_pre(const LR& la, const LR& lb, const RowGeom& g, int csa,
                                                  int csb, const uint4* __restrict__ lds, int chunks, int m,
                                                  const ChunkRegs (&fa)[NB], const ChunkRegs (&fb)[NB],
                                                  float (&ra)[MAXM], float (&rb)[MAXM]) {
#pragma unroll
  for (int r = 0; r < MAXM; ++r) ra[r] = rb[r] = 0.f;
  consume_pass_pair<FMT, NB, MAXM>(fa, fb, la.li, 0, g.l2, lds, chunks, m, ra, rb);
  const int passes = g.P / NB;
  for (int p = 1; p < passes; ++p) {
    ChunkRegs ca[NB], cb[NB];
    issue_pass<FMT, NB>(la, p, g.l2, csa, ca);
    issue_pass<FMT, NB>(lb, p, g.l2, csb, cb);
    consume_pass_pair<FMT, NB, MAXM>(ca, cb, la.li, p, g.l2, lds, chunks, m, ra, rb);
  }
#pragma unroll
  for (int r = 0; r < MAXM; ++r) {
    if (r < m) {
      ra[r] = group_sum(ra[r], g.l2);
      rb[r] = group_sum(rb[r], g.l2);
    }
  }
}

// Dispatches a callable on the compile-time pass width.
template <class F>
inline void dispatch_nb(int nb, F&& f) {
  switch (nb) {
    case 8: f(std::integral_constant<int, 8>{}); break;
    case 6: f(std::integral_constant<int, 6>{}); break;
    case 5: f(std::integral_constant<int, 5>{}); break;
    case 4: f(std::integral_constant<int, 4>{}); break;
    case 3: f(std::integral_constant<int, 3>{}); break;
    case 2: f(std::integral_constant<int, 2>{}); break;
    default: f(std::integral_constant<int, 1>{}); break;
  }
}

}  // namespace dgpp_amd
