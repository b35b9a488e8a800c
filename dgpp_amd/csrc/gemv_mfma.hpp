// The matrix-core form of the weight-streaming GEMV for gfx950: the same launchers, the same
// layouts in memory, but the dot products run on v_mfma_f32_16x16x32_bf16 instead of the vector
// ALU, so the per-weight vector work is the decode alone and up to 16 activation rows ride on one
// pass over the weights.
//
// Shape. A wavefront owns a ROW GROUP of 16 weight rows. Per STEP one load instruction reads 64
// contiguous bytes of each of the 16 rows (128 FP4 or 64 FP8 elements per row and step), 16 bytes
// per lane; after a lane permute lane (r = lane % 16, q = lane / 16) holds bytes q * 16 .. + 15 of
// row r's 64. The lane decodes its 16 bytes to bf16 in registers (hardware FP4 / FP8 conversions, block scale folded
// in) and feeds them, 8 elements at a time, as the A operand; the B operand is the matching 8
// activations of activation row (lane % 16), read as one 16-byte vector from an LDS stage laid
// out [8-element block][activation row]. D[weight row][activation row] accumulates in fp32: lane
// (r, q) ends up with weight rows 4q .. 4q+3 of activation row r.
//
// K is cut in PARTS (1, 2 or 4, a function of k alone): each part accumulates on its own and the
// parts are added in ascending order at the end. The decode-slot kernels give each part to its own
// wavefront (that is where a one-token batch gets its parallelism from); the dense and grouped
// kernels walk the parts one after the other with one accumulator each. Both therefore run the
// SAME arithmetic per (weight row, activation row): results do not depend on the launcher, the
// grid, or how many activation rows share the pass.
//
// Value semantics are the vector core's (gemv_core.hpp); NVFP4 weights are formed as
// bf16(e2m1 * e4m3), which is exact.
#pragma once

#include "gemv_core.hpp"

namespace dgpp_amd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

template <int FMT>
struct MTraits {
  static constexpr int kLoadElems = FmtTraits<FMT>::kElemsPerChunk;  // k elements of one 16-byte lane load
  static constexpr int kSub = kLoadElems / 8;                        // MFMA operands per lane load
  static constexpr int kStepElems = 4 * kLoadElems;                  // k elements per row and step
  static constexpr int kStepBlocks = 4 * kSub;                       // 8-element blocks per row and step
};

constexpr int kMaxParts = 4;
constexpr int kGroupRows = 16;       // weight rows of a row group
constexpr int kTileCols = 16;        // activation rows of one MFMA tile

struct MGeom {
  int parts;       // 1, 2 or 4
  int part_steps;  // steps per part, a multiple of 4 (trailing parts may be shorter or empty)
  int steps;       // steps covering k
};
template <int FMT>
__host__ __device__ inline MGeom mgeom(int k) {
  constexpr int se = MTraits<FMT>::kStepElems;
  MGeom g;
  g.parts = k >= 4096 ? 4 : (k >= 2048 ? 2 : 1);
  g.steps = (k + se - 1) / se;
  g.part_steps = ((g.steps + g.parts - 1) / g.parts + 3) & ~3;   // whole tiles of four steps
  return g;
}

union Frag {
  bf16x8_t v;
  bf16x2_t p[4];
};

// The MFMA A operands of one 16-byte lane load.
template <int FMT>
__device__ __forceinline__ void decode_frags(const ChunkRegs& ch, Frag (&f)[MTraits<FMT>::kSub]) {
  const uint32_t w[4] = {ch.w.x, ch.w.y, ch.w.z, ch.w.w};
  if constexpr (FMT == kFmtMxfp4) {
    const float s = bits_f32(ch.s << 23);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      f[q].p[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 0);
      f[q].p[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 1);
      f[q].p[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 2);
      f[q].p[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[q], s, 3);
    }
  } else if constexpr (FMT == kFmtNvfp4) {
    const float s0 = __builtin_amdgcn_cvt_f32_fp8(ch.s, 0);
    const float s1 = __builtin_amdgcn_cvt_f32_fp8(ch.s, 1);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float s = q < 2 ? s0 : s1;
      const f32x2_t v0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[q], 1.0f, 0);
      const f32x2_t v1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[q], 1.0f, 1);
      const f32x2_t v2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[q], 1.0f, 2);
      const f32x2_t v3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[q], 1.0f, 3);
      f[q].p[0] = pack_bf16(v0.x * s, v0.y * s);
      f[q].p[1] = pack_bf16(v1.x * s, v1.y * s);
      f[q].p[2] = pack_bf16(v2.x * s, v2.y * s);
      f[q].p[3] = pack_bf16(v3.x * s, v3.y * s);
    }
  } else if constexpr (FMT == kFmtFp8E8M0) {
    const float s = bits_f32(ch.s << 23);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      f[q].p[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * q], s, false);
      f[q].p[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * q], s, true);
      f[q].p[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * q + 1], s, false);
      f[q].p[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * q + 1], s, true);
    }
  } else {
    const float s = bits_f32(ch.s);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[2 * q + h], false);
        const f32x2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[2 * q + h], true);
        f[q].p[2 * h + 0] = pack_bf16(lo.x * s, lo.y * s);
        f[q].p[2 * h + 1] = pack_bf16(hi.x * s, hi.y * s);
      }
    }
  }
}

// The FP16 operands of an NVFP4 lane load, for kernels whose activations are FP16 as well (the W4A4 form: both
// operands are e2m1 x e4m3 products, six significant bits in [2^-10, 2688], exact in FP16). The scaled conversion
// applies the scale's exponent; its mantissa, 1 + m / 8, is one packed FP16 multiply per pair: 1.25 instructions
// per element against the 2 of the BF16 route (convert to f32, multiply, pack).
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
union FragH {
  f16x8_t v;
  f16x2_t p[4];
};
// (2^e, 1 + m / 8 in both halves) of an e4m3 scale given as f32: the conversion's scale operand and the multiplier.
__device__ __forceinline__ void split_scale_f16(float s, float& pow2, f16x2_t& mant) {
  const uint32_t bits = f32_bits(s);
  pow2 = bits_f32(bits & 0x7F800000u);
  const uint32_t h = ((bits >> 13) & 0x0380u) | 0x3C00u;
  mant = __builtin_bit_cast(f16x2_t, h | (h << 16));
}
__device__ __forceinline__ void decode_frags_nvfp4_f16(const ChunkRegs& ch, FragH (&f)[4]) {
  const uint32_t w[4] = {ch.w.x, ch.w.y, ch.w.z, ch.w.w};
  float e0, e1;
  f16x2_t m0, m1;
  split_scale_f16(__builtin_amdgcn_cvt_f32_fp8(ch.s, 0), e0, m0);
  split_scale_f16(__builtin_amdgcn_cvt_f32_fp8(ch.s, 1), e1, m1);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float e = q < 2 ? e0 : e1;
    const f16x2_t m = q < 2 ? m0 : m1;
    f[q].p[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[q], e, 0) * m;
    f[q].p[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[q], e, 1) * m;
    f[q].p[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[q], e, 2) * m;
    f[q].p[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[q], e, 3) * m;
  }
}
__device__ __forceinline__ f32x4_t mfma_f16(const FragH& a, const uint4& b, f32x4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, __builtin_bit_cast(f16x8_t, b), acc, 0, 0, 0);
}

__device__ __forceinline__ f32x4_t mfma_bf16(const Frag& a, const uint4& b, f32x4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
}

// Per-lane LOAD addressing of a row group starting at row0. Loads are issued row-major — lane l reads
// piece l % 4 of row l / 4, so a quarter wavefront touches 4 rows x 64 contiguous bytes instead of 16
// rows x 16 bytes — and a lane permute (to_operand_layout) then hands lane (r, q) = r + 16 q the 16
// bytes of row r, piece q that the matrix core expects from it.
struct GroupLane {
  const uint8_t* payload_row;
  const void* scale_row;
  int q;          // the piece this lane LOADS
  int from;       // byte address (lane * 4) of the lane whose load this lane consumes
};
template <bool NT>
struct GroupLaneT : GroupLane {
  static constexpr bool kNT = NT;   // load_chunk's load policy, part of the type
};
template <int FMT, bool NT = true>
__device__ __forceinline__ GroupLaneT<NT> group_lane(const MatRef& mat, int row0, int n, int k) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = row0 + (lane >> 2);
  const int r = row < n ? row : n - 1;   // rows past the end redo the last row; their results are dropped
  GroupLaneT<NT> gl;
  gl.q = lane & 3;
  gl.from = (4 * (lane & 15) + (lane >> 4)) * 4;
  if constexpr (FMT == kFmtFp8F32 || FMT == kFmtFp8E8M0) {
    gl.payload_row = mat.payload + static_cast<size_t>(r) * k;
    const size_t scale_cols = (static_cast<size_t>(k) + (1u << mat.cs) - 1) >> mat.cs;
    const size_t esz = FMT == kFmtFp8F32 ? 4 : 1;
    gl.scale_row = reinterpret_cast<const uint8_t*>(mat.scales) + (static_cast<size_t>(r >> mat.rs) * scale_cols) * esz;
  } else {
    gl.payload_row = mat.payload + static_cast<size_t>(r) * (k / 2);
    gl.scale_row = reinterpret_cast<const uint8_t*>(mat.scales) +
                   static_cast<size_t>(r) * (k / (FMT == kFmtNvfp4 ? 16 : 32));
  }
  return gl;
}

// The lane's 16 bytes of step `step` (chunk index step * 4 + q of the row), or zeros past k.
template <int FMT, class GL>
__device__ __forceinline__ void load_step(const GL& gl, int step, int chunks, int cs, ChunkRegs& out) {
  const int c = step * 4 + gl.q;
  if (c < chunks) {
    load_chunk<FMT, GL::kNT>(gl.payload_row, gl.scale_row, c, cs, out);
  } else {
    out.w = make_uint4(0u, 0u, 0u, 0u);   // code 0 is +0 in e2m1 and e4m3
    out.s = 0u;
  }
}

__device__ __forceinline__ void to_operand_layout(const GroupLane& gl, ChunkRegs& r) {
  r.w.x = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(gl.from, static_cast<int>(r.w.x)));
  r.w.y = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(gl.from, static_cast<int>(r.w.y)));
  r.w.z = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(gl.from, static_cast<int>(r.w.z)));
  r.w.w = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(gl.from, static_cast<int>(r.w.w)));
  r.s = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(gl.from, static_cast<int>(r.s)));
}

// ---- row-wide tile loads -------------------------------------------------------------------------------
// The operand layout wants 16 different rows in 16 adjacent lanes; loading that way makes every quarter
// wavefront touch 4 - 16 rows with 64 or 16 bytes each, which the vector memory pipe serves well below its
// streaming rate. The block kernels therefore load a TILE — 16 rows x 256 bytes, the four steps of a chunk —
// row-major (instruction i reads rows 4i .. 4i+3, sixteen lanes per row: 256 contiguous bytes per quarter
// wavefront), park it in a wavefront-private LDS region and read it back in operand layout. The region is
// XOR-swizzled by row so that both the row-major writes and the column-major reads are conflict-free.
constexpr int kTileUnits = 256;   // 16-byte units of one tile (4 KB)

struct WideLane {
  const uint8_t* base;   // matrix payload
  uint32_t off[4];       // byte offset of this lane's row for each of the four load instructions
  uint32_t row_bytes;
  int piece;             // 16-byte piece of the 256-byte row segment this lane loads
};
template <int FMT>
__device__ __forceinline__ WideLane wide_lane(const MatRef& mat, int row0, int n, int k) {
  const int lane = threadIdx.x & (kWave - 1);
  WideLane w;
  w.base = mat.payload;
  w.row_bytes = static_cast<uint32_t>(FmtTraits<FMT>::kIsFp4 ? k / 2 : k);
  w.piece = lane & 15;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = row0 + 4 * i + (lane >> 4);
    w.off[i] = static_cast<uint32_t>(row < n ? row : n - 1) * w.row_bytes;   // rows past the end redo the last row
  }
  return w;
}
// The tile that starts at step `step0` (bytes step0 * 64 ... + 255 of each row); zeros past the row's end.
template <bool NT>
__device__ __forceinline__ void issue_tile(const WideLane& w, int step0, uint4 (&t)[4]) {
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  const uint32_t in_row = static_cast<uint32_t>(step0) * 64u + static_cast<uint32_t>(w.piece) * 16u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (in_row < w.row_bytes) {
      const __attribute__((address_space(1))) u32x4_t* src =
          (const __attribute__((address_space(1))) u32x4_t*)(uintptr_t)(w.base + w.off[i] + in_row);
      const u32x4_t v = NT ? __builtin_nontemporal_load(src) : *src;
      t[i] = make_uint4(v.x, v.y, v.z, v.w);
    } else {
      t[i] = make_uint4(0u, 0u, 0u, 0u);
    }
  }
}
__device__ __forceinline__ void commit_tile(uint4* __restrict__ region, const uint4 (&t)[4]) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * i + (lane >> 4);
    region[r * 16 + ((lane & 15) ^ r)] = t[i];
  }
}
// Lane (r = lane % 16, q = lane / 16): its 16 bytes of step t of the tile (piece 4 t + q of row r).
__device__ __forceinline__ uint4 tile_operand(const uint4* __restrict__ region, int t) {
  const int lane = threadIdx.x & (kWave - 1);
  const int r = lane & 15;
  return region[r * 16 + ((4 * t + (lane >> 4)) ^ r)];
}

// The block scales of a row group in operand layout (lane (r, q): row r, piece q of a step).
struct ScaleLane {
  const void* scale_row;
  int q;
};
template <int FMT>
__device__ __forceinline__ ScaleLane scale_lane(const MatRef& mat, int row0, int n, int k) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = row0 + (lane & 15);
  const int r = row < n ? row : n - 1;
  ScaleLane sl;
  sl.q = lane >> 4;
  if constexpr (FMT == kFmtFp8F32 || FMT == kFmtFp8E8M0) {
    const size_t scale_cols = (static_cast<size_t>(k) + (1u << mat.cs) - 1) >> mat.cs;
    const size_t esz = FMT == kFmtFp8F32 ? 4 : 1;
    sl.scale_row = reinterpret_cast<const uint8_t*>(mat.scales) + (static_cast<size_t>(r >> mat.rs) * scale_cols) * esz;
  } else {
    sl.scale_row = reinterpret_cast<const uint8_t*>(mat.scales) + static_cast<size_t>(r) * (k / (FMT == kFmtNvfp4 ? 16 : 32));
  }
  return sl;
}
// ChunkRegs::s of the lane's piece of step `step` (0 past k).
template <int FMT>
__device__ __forceinline__ uint32_t load_scale(const ScaleLane& sl, int step, int chunks, int cs) {
  const int c = step * 4 + sl.q;
  if (c >= chunks) return 0u;
#define DGPP_AS1 __attribute__((address_space(1)))
  if constexpr (FMT == kFmtFp8F32) {
    return ((const DGPP_AS1 uint32_t*)(uintptr_t)sl.scale_row)[(c * 16) >> cs];
  } else if constexpr (FMT == kFmtFp8E8M0) {
    return ((const DGPP_AS1 uint8_t*)(uintptr_t)sl.scale_row)[(c * 16) >> cs];
  } else if constexpr (FMT == kFmtNvfp4) {
    return ((const DGPP_AS1 uint16_t*)(uintptr_t)sl.scale_row)[c];
  } else {
    return ((const DGPP_AS1 uint8_t*)(uintptr_t)sl.scale_row)[c];
  }
#undef DGPP_AS1
}

// acc += the chunk whose tile sits in `region` (operand reads) with block scales sc[0 .. 3]; `valid` steps.
// H16: the stage holds FP16 activations and the weights decode to FP16 (NVFP4 only).
template <int FMT, bool H16 = false>
__device__ __forceinline__ void mfma_tile(const uint4* __restrict__ region, const uint32_t (&sc)[4],
                                          const uint4* __restrict__ lane_stage, int m, int valid, f32x4_t& acc) {
  constexpr int kSub = MTraits<FMT>::kSub;
  static_assert(!H16 || FMT == kFmtNvfp4, "the FP16 route decodes NVFP4");
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i < valid) {
      ChunkRegs ch;
      ch.w = tile_operand(region, i);
      ch.s = sc[i];
      if constexpr (H16) {
        FragH f[4];
        decode_frags_nvfp4_f16(ch, f);
#pragma unroll
        for (int j = 0; j < kSub; ++j) acc = mfma_f16(f[j], lane_stage[(i * 4 * kSub + j) * m], acc);
      } else {
        Frag f[kSub];
        decode_frags<FMT>(ch, f);
#pragma unroll
        for (int j = 0; j < kSub; ++j) acc = mfma_bf16(f[j], lane_stage[(i * 4 * kSub + j) * m], acc);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// One 8-element block of an activation row as a 16-byte vector; zeros past k.
__device__ __forceinline__ uint4 load_act_block(const uint16_t* __restrict__ row, int k0, int k, bool aligned) {
  if (k0 >= k) return make_uint4(0u, 0u, 0u, 0u);
  if (aligned) return *reinterpret_cast<const uint4*>(row + k0);
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = static_cast<uint32_t>(row[k0 + 2 * i]) | (static_cast<uint32_t>(row[k0 + 2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// acc += sum over the NB steps of `regs` (steps step0 ... relative to the stage at `stage`):
// stage unit of (step t, lane q, sub j, activation row c) is ((t * 4 + q) * kSub + j) * m + c.
// Only the first `valid` steps of the chunk exist (the rest hold zeros and their stage units may
// never have been written, so they must not reach the matrix core).
template <int FMT, int NB>
__device__ __forceinline__ void mfma_chunk(const GroupLane& gl, ChunkRegs (&regs)[NB], const uint4* __restrict__ lane_stage,
                                           int m, int valid, f32x4_t& acc) {
  constexpr int kSub = MTraits<FMT>::kSub;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if (i < valid) {
      to_operand_layout(gl, regs[i]);
      Frag f[kSub];
      decode_frags<FMT>(regs[i], f);
#pragma unroll
      for (int j = 0; j < kSub; ++j) acc = mfma_bf16(f[j], lane_stage[(i * 4 * kSub + j) * m], acc);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}
template <int FMT, int NB>
__device__ __forceinline__ void mfma_chunk_pair(const GroupLane& gl, ChunkRegs (&ra)[NB], ChunkRegs (&rb)[NB],
                                                const uint4* __restrict__ lane_stage, int m, int valid,
                                                f32x4_t& acc_a, f32x4_t& acc_b) {
  constexpr int kSub = MTraits<FMT>::kSub;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if (i < valid) {
      to_operand_layout(gl, ra[i]);
      to_operand_layout(gl, rb[i]);
      Frag fa[kSub], fb[kSub];
      decode_frags<FMT>(ra[i], fa);
      decode_frags<FMT>(rb[i], fb);
#pragma unroll
      for (int j = 0; j < kSub; ++j) {
        const uint4 b = lane_stage[(i * 4 * kSub + j) * m];
        acc_a = mfma_bf16(fa[j], b, acc_a);
        acc_b = mfma_bf16(fb[j], b, acc_b);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

}  // namespace dgpp_amd
