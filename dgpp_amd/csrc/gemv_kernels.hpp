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
#include "router_select.hpp"
#include "swiglu.hpp"

namespace dgpp_amd {

// Every GEMV kernel is compiled for at least this many resident wavefronts per SIMD (a cap of 128
// VGPRs): the streams are latency-bound, and the compiler otherwise trades occupancy for hoisting
// every decode of a pass ahead of the first dot.
#ifndef DGPP_MIN_WAVES_PER_SIMD
#define DGPP_MIN_WAVES_PER_SIMD 2
#endif
constexpr int kMinWavesPerSimd = DGPP_MIN_WAVES_PER_SIMD;

// ---- epilogues (SwiGLU: swiglu.hpp) -------------------------------------------------------------
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
  int once;                 // all m rows ride on one pass over the weights (nontemporal loads)
  // matrix-core form only: the activation is SwiGLU(act, act_up) with this clamp, computed as the rows are staged
  const uint16_t* act_up = nullptr;
  float limit = 0.f;
  // matrix-core form, NVFP4 only: `act` holds NVFP4 activation codes (act_stride in BYTES) with these scale rows and
  // per-row globals (the W4A4 form)
  const uint8_t* a4_scales = nullptr;
  size_t a4_scale_stride = 0;
  const float* a4_gs = nullptr;
};

template <int FMT, int MAXR, int NB, bool NT>
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
    const auto lr = lane_row<FMT, NT>(a.mat, row0, a.n, a.k, g.l2);
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

// Up to four dense problems of one k and one row count in ONE launch (reference: launch_scale_gemv_multi_bf16,
// src/kernels/scale_gemm.cu:625-672): the grid is the problems' row tiles laid end to end; a block finds its problem
// and then does what gemv_dense_kernel does for it, so each output is bitwise its single launch's.
constexpr int kMaxDenseProblems = 4;
struct DenseMultiArgs {
  DenseArgs p[kMaxDenseProblems];
  int tile_end[kMaxDenseProblems];   // one past the last grid block of each problem
  int count;
};

template <int FMT, int MAXR, int NB, bool NT>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void gemv_dense_multi_kernel(DenseMultiArgs ma, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  int which = 0;
  const int b = static_cast<int>(blockIdx.x);
#pragma unroll
  for (int i = 0; i + 1 < kMaxDenseProblems; ++i)
    if (i + 1 < ma.count && b >= ma.tile_end[i]) which = i + 1;
  const DenseArgs& a = ma.p[which];
  const int bx = b - (which ? ma.tile_end[which - 1] : 0);
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  stage_activations<FMT>(a.act, a.act_stride, a.m, a.k, lds);
  __syncthreads();
  const float divisor = load_divisor<FMT>(a.global);
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  int row0 = bx * block_rows(g, steps) + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const auto lr = lane_row<FMT, NT>(a.mat, row0, a.n, a.k, g.l2);
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
// Activation vectors (16 bytes) a thread holds between the issue and the commit of a split stage.
constexpr int kSplitStageVecs = 2;

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
  int match;                // no order and tokens * top_k <= 64: find the slots that share an expert by ballot
  int once;                 // few slots can share an expert: the weights stream through once (nontemporal loads)
  int want_shared;          // 0: routed slots, 1: shared slots (others exit)
  int shared_view_base;     // >= 0: shared matrices come from views[base + which]
  // Down launches of the shared slots only, nullable: the token's accumulation as the epilogue. `out` then holds the
  // routed slots' finished rows; the shared row is not stored, the token's row goes to acc_out as bf16:
  // a = 0; a = fma(w_j, out[slot j], a) for j ascending; a = fma(1, shared dot, a); one rounding.
  const float* acc_weights; // [tokens, top_k]
  uint16_t* acc_out;        // [tokens, n]
};

// The router selection a gate/up launch can repeat in every block instead of reading `ids` (select_gate_up_kernel).
struct SelectArgs {
  const float* scores;      // [tokens, n_experts]
  const float* biased;      // [tokens, n_experts]
  int32_t* ids;             // out [tokens, top_k], stored by block (0, 0)
  float* weights;           // out [tokens, top_k]
  int mode;                 // DGPP_ROUTER_*
  int n_experts;
  float scaling;
  int norm_topk;
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

// The slots one block serves: a RUN of up to MAXM slots that follow each other in `order` and use
// the same expert (the order sorts slots by expert; the shared slots of all tokens form one run).
// The expert's rows are then read once for the whole run. A position is the run's leader when the
// count of same-expert positions right before it is a multiple of MAXM; other blocks exit.
template <int MAXM>
struct SlotRun {
  int m;
  int slot[MAXM];
  int token[MAXM];
  int view_base;   // index of the expert's gate view, or < 0: matrices from the launch arguments
};

// Expert key of a logical slot (-1 for the shared slot) and its token.
__device__ __forceinline__ int slot_key(const SlotArgs& a, int slot, int& token) {
  token = slot / (a.top_k + 1);
  const int j = slot - token * (a.top_k + 1);
  return j == a.top_k ? -1 : a.ids[static_cast<size_t>(token) * a.top_k + j];
}

template <int MAXM>
__device__ __forceinline__ bool resolve_run_at(const SlotArgs& a, SlotRun<MAXM>& run, int p) {
  if (p >= a.slots) return false;
  const int slot0 = a.order ? a.order[p] : p;
  int token0;
  const int key0 = slot_key(a, slot0, token0);
  if ((key0 < 0) != (a.want_shared != 0)) return false;
  run.m = 1;
  run.slot[0] = slot0;
  run.token[0] = token0;
  run.view_base = key0 < 0 ? a.shared_view_base : key0 * 3;
  if constexpr (MAXM > 1) {
    if (a.order) {
      int back = 0, t;
      while (p - back - 1 >= 0 && slot_key(a, a.order[p - back - 1], t) == key0) ++back;
      if (back % MAXM != 0) return false;
      bool alive = true;
#pragma unroll
      for (int r = 1; r < MAXM; ++r) {
        run.slot[r] = slot0;
        run.token[r] = token0;
        if (alive && p + r < a.slots) {
          const int s = a.order[p + r];
          if (slot_key(a, s, t) == key0) {
            run.slot[r] = s;
            run.token[r] = t;
            run.m = r + 1;
          } else {
            alive = false;
          }
        } else {
          alive = false;
        }
      }
    } else if (a.match && key0 >= 0) {
      // No order given, a small decode batch (tokens * top_k <= 128): the slots that use this expert are found
      // with two ballots over the routed ids (an expert occurs at most once per token, so they sit in
      // different tokens). The first of every MAXM of them, in (token, j) order, leads the run.
      const int lane = threadIdx.x & (kWave - 1);
      const int tk = (a.slots / (a.top_k + 1)) * a.top_k;
      const int lo = lane < tk ? a.ids[lane] : -1;
      const int hi = lane + kWave < tk ? a.ids[lane + kWave] : -1;
      const unsigned long long m0 = __builtin_amdgcn_ballot_w64(lo == key0);
      const unsigned long long m1 = __builtin_amdgcn_ballot_w64(hi == key0);
      const int mine = token0 * a.top_k + (slot0 - token0 * (a.top_k + 1));
      auto below = [](unsigned long long m, int n) {   // set bits of m at positions < n, n in 0 .. 64
        return n <= 0 ? 0 : __builtin_popcountll(n >= 64 ? m : m & ((1ull << n) - 1ull));
      };
      const int before = below(m0, mine) + below(m1, mine - kWave);
      if (before % MAXM != 0) return false;
      auto next_after = [&](int at) {                  // the next sharer's index above `at`, or -1
        if (at < kWave - 1) {
          const unsigned long long r = m0 >> (at + 1);
          if (r != 0ull) return at + 1 + __builtin_ctzll(r);
        }
        const int from = at < kWave ? 0 : at - kWave + 1;
        if (from < kWave) {
          const unsigned long long r = m1 >> from;
          if (r != 0ull) return kWave + from + __builtin_ctzll(r);
        }
        return -1;
      };
      int at = mine;
      bool alive = true;
#pragma unroll
      for (int r = 1; r < MAXM; ++r) {
        run.slot[r] = slot0;
        run.token[r] = token0;
        const int nxt = alive ? next_after(at) : -1;
        if (nxt >= 0) {
          at = nxt;
          const int t = at / a.top_k;
          run.slot[r] = t * (a.top_k + 1) + (at - t * a.top_k);
          run.token[r] = t;
          run.m = r + 1;
        } else {
          alive = false;
        }
      }
    } else if (a.match) {
      // The shared slots of consecutive tokens use the same (shared) expert.
      const int tokens = a.slots / (a.top_k + 1);
      if (token0 % MAXM != 0) return false;
#pragma unroll
      for (int r = 1; r < MAXM; ++r) {
        const bool have = token0 + r < tokens;
        run.token[r] = have ? token0 + r : token0;
        run.slot[r] = run.token[r] * (a.top_k + 1) + a.top_k;
        if (have) run.m = r + 1;
      }
    }
  }
  return true;
}
template <int MAXM>
__device__ __forceinline__ bool resolve_run(const SlotArgs& a, SlotRun<MAXM>& run) {
  return resolve_run_at<MAXM>(a, run, static_cast<int>(blockIdx.y));
}

// What a gate/up block of the one-launch chain (gemv_chain.hpp) does beyond storing its act values: the values go
// out as agent-scope stores (written through to where every XCD reads them) and, once every wavefront's stores
// have been acknowledged, one thread counts the block in on the readiness word of each slot it served.
struct SlotPublish {
  unsigned* ready;   // one word per routed slot (index token * top_k + j), `stride` words apart
  int stride;
  unsigned wrap;     // the word goes back to zero after wrap + 1 increments
};

// `p` names the block's position (its slot, or its place in `order`), `tile` its row tile. WAVES wavefronts per
// block; PUBLISH: the chain form above.
template <int FMT, int NB, int MAXM, bool SPLIT, bool NT, int WAVES = kWavesPerBlock, bool PUBLISH = false>
__device__ __forceinline__ void slot_gate_up_body(const SlotArgs& a, const RowGeom& g, int steps, uint4* __restrict__ lds,
                                                  int p, int tile, const SlotPublish* pub = nullptr) {
  constexpr int kThreads = WAVES * kWave;
  SlotRun<MAXM> run;
  if (!resolve_run_at<MAXM>(a, run, p)) return;
  const int rpw = kWave >> g.l2;
  const int rows_per_block = WAVES * rpw * steps;
  if (tile * rows_per_block >= a.n) return;
  MatRef mg, mu;
  const float *gg = nullptr, *gu = nullptr;
  if (run.view_base >= 0) {
    mg = mat_of_view<FMT>(a.views[run.view_base + 0], &gg);
    mu = mat_of_view<FMT>(a.views[run.view_base + 1], &gu);
  } else {
    mg = a.sh[0];
    mu = a.sh[1];
  }
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  const int row_vecs = FmtTraits<FMT>::kPieces * chunks;
  const int wave = threadIdx.x >> 6;
  int row0 = tile * rows_per_block + wave * rpw;
  uint16_t* act = static_cast<uint16_t*>(a.out);
  // Fast set-up (rows of at most 4096 aligned elements): activation loads, then the first step's weight
  // loads, then the LDS commit and the barrier — the weights travel while the block sets up.
  constexpr int XV = (kSplitStageVecs * kBlockThreads + kThreads - 1) / kThreads;
  const auto lg = lane_row<FMT, NT>(mg, row0, a.n, a.k, g.l2);
  const auto lu = lane_row<FMT, NT>(mu, row0, a.n, a.k, g.l2);
  ChunkRegs fg[NB], fu[NB];
  if constexpr (SPLIT) {
    StageRegs<XV> xr[MAXM];
#pragma unroll
    for (int r = 0; r < MAXM; ++r)   // every register set is loaded (unused run entries repeat row 0): no partial state
      stage_issue<FMT, XV>(a.x + static_cast<size_t>(run.token[r]) * a.x_stride, a.k, threadIdx.x, kThreads, xr[r]);
    issue_pass<FMT, NB>(lg, 0, g.l2, mg.cs, fg);
    issue_pass<FMT, NB>(lu, 0, g.l2, mu.cs, fu);
#pragma unroll
    for (int r = 0; r < MAXM; ++r)
      if (r < run.m) stage_commit<FMT, XV>(xr[r], a.k, threadIdx.x, kThreads, lds + r * row_vecs);
  } else {
#pragma unroll
    for (int r = 0; r < MAXM; ++r)
      if (r < run.m)
        stage_activations<FMT>(a.x + static_cast<size_t>(run.token[r]) * a.x_stride, a.x_stride, 1, a.k, lds + r * row_vecs);
  }
  __syncthreads();
  const float dg = load_divisor<FMT>(gg), du = load_divisor<FMT>(gu);
  auto finish = [&](const LaneRow& l, const float (&ag)[MAXM], const float (&au)[MAXM]) {
    if (l.li == 0 && l.row < a.n) {
#pragma unroll
      for (int r = 0; r < MAXM; ++r)
        if (r < run.m) {
          const uint16_t v = swiglu_bf16(finish_dot<FMT>(ag[r], dg), finish_dot<FMT>(au[r], du), a.limit);
          uint16_t* at = act + static_cast<size_t>(run.slot[r]) * a.out_stride + l.row;
          if constexpr (PUBLISH) __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          else *at = v;
        }
    }
  };
  int s = 0;
  if constexpr (SPLIT) {
    if (row0 < a.n) {
      float ag[MAXM], au[MAXM];
      row_dots_pair_pre<FMT, NB, MAXM>(lg, lu, g, mg.cs, mu.cs, lds, chunks, run.m, fg, fu, ag, au);
      finish(lg, ag, au);
    }
    s = 1;
    row0 += WAVES * rpw;
  }
  for (; s < steps; ++s, row0 += WAVES * rpw) {
    if (row0 >= a.n) break;
    const auto l2g = lane_row<FMT, NT>(mg, row0, a.n, a.k, g.l2);
    const auto l2u = lane_row<FMT, NT>(mu, row0, a.n, a.k, g.l2);
    float ag[MAXM], au[MAXM];
    row_dots_pair<FMT, NB, MAXM>(l2g, l2u, g, mg.cs, mu.cs, lds, chunks, run.m, ag, au);
    finish(l2g, ag, au);
  }
  if constexpr (PUBLISH) {
    // vmcnt(0): every act store of this wavefront has been acknowledged by the memory side (a block barrier alone
    // does not wait for outstanding stores); then the block is counted in, once per slot of its run.
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#pragma unroll
    for (int r = 0; r < MAXM; ++r)
      if (r < run.m && static_cast<int>(threadIdx.x) == r)
        atomicInc(pub->ready + static_cast<size_t>(run.slot[r] - run.token[r]) * pub->stride, pub->wrap);
  }
}

template <int FMT, int NB, int MAXM, bool SPLIT, bool NT>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_gate_up_kernel(SlotArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  slot_gate_up_body<FMT, NB, MAXM, SPLIT, NT>(a, g, steps, lds, static_cast<int>(blockIdx.y), static_cast<int>(blockIdx.x));
}

// ---- gate / up in different formats (the per-projection form) -------------------------------------------------------
// One projection of every routed expert is block-FP8 (its table entry's payload / scales / shifts), the other NVFP4
// (payload / fp4_scales / fp4_global); GATE_FP4 says which (reference: src/kernels/glm_moe.cu:4882-4922). A block takes
// a tile of rows of ONE slot: the token's row is staged twice, in each core's LDS order; the wavefronts walk the
// tile's rows of the FP8 matrix with the FP8 core, then of the FP4 matrix with the FP4 core (each with its own row
// geometry: row_dots, the uniform kernels' chain per row, bit for bit), park the finished dots in LDS, and the SwiGLU
// runs on the pairs with the uniform kernels' rounding points.
template <int NB8, int NB4, bool GATE_FP4>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_gate_up_mixed_kernel(SlotArgs a, RowGeom g8, RowGeom g4,
                                                                                            int rows_per_block) {
  extern __shared__ uint4 lds[];
  SlotRun<1> run;
  if (!resolve_run<1>(a, run)) return;
  const int tile_row0 = static_cast<int>(blockIdx.x) * rows_per_block;
  if (tile_row0 >= a.n) return;
  const DgppMoeExpertView& v8 = a.views[run.view_base + (GATE_FP4 ? 1 : 0)];
  const DgppMoeExpertView& v4 = a.views[run.view_base + (GATE_FP4 ? 0 : 1)];
  const float *unused = nullptr, *global4 = nullptr;
  const MatRef m8 = mat_of_view<kFmtFp8F32>(v8, &unused);
  const MatRef m4 = mat_of_view<kFmtNvfp4>(v4, &global4);
  const int row_vecs = a.k / 8;
  uint4* x8 = lds;
  uint4* x4 = lds + row_vecs;
  float* d8 = reinterpret_cast<float*>(lds + 2 * row_vecs);   // [rows_per_block] each
  float* d4 = d8 + rows_per_block;
  const uint16_t* x = a.x + static_cast<size_t>(run.token[0]) * a.x_stride;
  stage_activations<kFmtFp8F32>(x, a.x_stride, 1, a.k, x8);
  stage_activations<kFmtNvfp4>(x, a.x_stride, 1, a.k, x4);
  __syncthreads();
  const int wave = threadIdx.x >> 6;
  const int tile_end = min(a.n, tile_row0 + rows_per_block);
  {
    const int rpw = kWave >> g8.l2, chunks = a.k / FmtTraits<kFmtFp8F32>::kElemsPerChunk;
    for (int row0 = tile_row0 + wave * rpw; row0 < tile_end; row0 += kWavesPerBlock * rpw) {
      const auto lr = lane_row<kFmtFp8F32, false>(m8, row0, a.n, a.k, g8.l2);
      float acc[1];
      row_dots<kFmtFp8F32, 1, NB8>(lr, g8, m8.cs, x8, chunks, 1, acc);
      if (lr.li == 0 && lr.row < tile_end) d8[lr.row - tile_row0] = finish_dot<kFmtFp8F32>(acc[0], 1.0f);
    }
  }
  {
    const float divisor = load_divisor<kFmtNvfp4>(global4);
    const int rpw = kWave >> g4.l2, chunks = a.k / FmtTraits<kFmtNvfp4>::kElemsPerChunk;
    for (int row0 = tile_row0 + wave * rpw; row0 < tile_end; row0 += kWavesPerBlock * rpw) {
      const auto lr = lane_row<kFmtNvfp4, false>(m4, row0, a.n, a.k, g4.l2);
      float acc[1];
      row_dots<kFmtNvfp4, 1, NB4>(lr, g4, m4.cs, x4, chunks, 1, acc);
      if (lr.li == 0 && lr.row < tile_end) d4[lr.row - tile_row0] = finish_dot<kFmtNvfp4>(acc[0], divisor);
    }
  }
  __syncthreads();
  uint16_t* act = static_cast<uint16_t*>(a.out) + static_cast<size_t>(run.slot[0]) * a.out_stride;
  for (int r = threadIdx.x; tile_row0 + r < tile_end; r += kBlockThreads)
    act[tile_row0 + r] = GATE_FP4 ? swiglu_bf16(d4[r], d8[r], a.limit) : swiglu_bf16(d8[r], d4[r], a.limit);
}

// The router's selection and the routed gate/up pass of a ONE-token decode step in one launch: the first
// wavefront of every block repeats the selection (whole score row in registers: the selection kernel's own
// code), the ids go to LDS behind the activation stage and the block goes on as slot_gate_up_kernel does.
// Block (0, 0) stores ids and weights for the launches that follow. One token only: the repeated selection
// costs every SIMD a few microseconds per token, which a launch of its own undercuts from two tokens on.
// n_experts <= 512, routed slots only; the fast set-up, nontemporal weight loads.
template <int FMT, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void select_gate_up_kernel(SlotArgs a, SelectArgs sel, RowGeom g,
                                                                                        int steps) {
  extern __shared__ uint4 lds[];
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  int32_t* ids = reinterpret_cast<int32_t*>(lds + FmtTraits<FMT>::kPieces * chunks);
  const int lane = threadIdx.x & (kWave - 1);
  if (threadIdx.x < kWave) {
    int id;
    float w;
    if (sel.n_experts <= 4 * kWave) {
      if (sel.mode == DGPP_ROUTER_SOFTMAX_TOPK)
        rsel::select_token<DGPP_ROUTER_SOFTMAX_TOPK, 4>(sel.scores, sel.biased, sel.n_experts, a.top_k, sel.scaling, sel.norm_topk, lane, id, w);
      else
        rsel::select_token<DGPP_ROUTER_SIGMOID_BIAS, 4>(sel.scores, sel.biased, sel.n_experts, a.top_k, sel.scaling, sel.norm_topk, lane, id, w);
    } else {
      if (sel.mode == DGPP_ROUTER_SOFTMAX_TOPK)
        rsel::select_token<DGPP_ROUTER_SOFTMAX_TOPK, 8>(sel.scores, sel.biased, sel.n_experts, a.top_k, sel.scaling, sel.norm_topk, lane, id, w);
      else
        rsel::select_token<DGPP_ROUTER_SIGMOID_BIAS, 8>(sel.scores, sel.biased, sel.n_experts, a.top_k, sel.scaling, sel.norm_topk, lane, id, w);
    }
    if (lane < a.top_k) {
      ids[lane] = id;
      if (blockIdx.x == 0 && blockIdx.y == 0) {
        sel.ids[lane] = id;
        sel.weights[lane] = w;
      }
    }
  }
  __syncthreads();
  SlotArgs b = a;
  b.ids = ids;
  slot_gate_up_body<FMT, NB, 1, true, true>(b, g, steps, lds, static_cast<int>(blockIdx.y), static_cast<int>(blockIdx.x));
}

// Down rows of a run of slots, unrounded f32.
template <int FMT, int NB, int MAXM, bool NT, bool ACC = false>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void slot_down_kernel(SlotArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  SlotRun<MAXM> run;
  if (!resolve_run<MAXM>(a, run)) return;
  const int rows_per_block = block_rows(g, steps);
  const int tile_row0 = static_cast<int>(blockIdx.x) * rows_per_block;
  if (tile_row0 >= a.n) return;
  MatRef md;
  const float* gd = nullptr;
  if (run.view_base >= 0)
    md = mat_of_view<FMT>(a.views[run.view_base + 2], &gd);
  else
    md = a.sh[0];
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  const int row_vecs = FmtTraits<FMT>::kPieces * chunks;
  // The down projection consumes each slot's own activation row.
#pragma unroll
  for (int r = 0; r < MAXM; ++r)
    if (r < run.m)
      stage_activations<FMT>(a.x + static_cast<size_t>(run.slot[r]) * a.x_stride, a.x_stride, 1, a.k, lds + r * row_vecs);
  __syncthreads();
  const float dd = load_divisor<FMT>(gd);
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  float* out = static_cast<float*>(a.out);
  int row0 = tile_row0 + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const auto lr = lane_row<FMT, NT>(md, row0, a.n, a.k, g.l2);
    float acc[MAXM];
    row_dots<FMT, MAXM, NB>(lr, g, md.cs, lds, chunks, run.m, acc);
    if (lr.li == 0 && lr.row < a.n) {
      if constexpr (ACC) {
#pragma unroll
        for (int r = 0; r < MAXM; ++r)
          if (r < run.m) {
            const int t = run.token[r];
            const size_t base = static_cast<size_t>(t) * (a.top_k + 1);
            float v = 0.f;
            for (int j = 0; j < a.top_k; ++j)
              v = fmaf(a.acc_weights[static_cast<size_t>(t) * a.top_k + j], out[(base + j) * a.out_stride + lr.row], v);
            v = fmaf(1.0f, finish_dot<FMT>(acc[r], dd), v);
            a.acc_out[static_cast<size_t>(t) * a.n + lr.row] = f32_to_bf16(v);
          }
      } else {
#pragma unroll
        for (int r = 0; r < MAXM; ++r)
          if (r < run.m) out[static_cast<size_t>(run.slot[r]) * a.out_stride + lr.row] = finish_dot<FMT>(acc[r], dd);
      }
    }
  }
}

// ---- decode: routed down projection + ordered accumulation, token-major ----------------------------------
// One block per (row tile, token), one wavefront per routed slot of the token: wavefront j streams the tile's
// rows of expert ids[t, j]'s down matrix against the slot's own activation row (the slot kernels' chain per
// row, bit for bit), the top_k partial rows meet in LDS and the token's accumulation chain
// (a = 0; a = fma(w_j, y_j, a), j ascending; one rounding) runs right there: no [slots, n] round trip
// through memory and no second launch. Routed slots only (no shared expert in the chain).
struct TokenDownArgs {
  const uint16_t* act;      // [slots, act_stride] slot activation rows, slot = t * (top_k + 1) + j
  size_t act_stride;
  const int32_t* ids;       // [tokens, top_k]
  const DgppMoeExpertView* views;
  const float* weights;     // [tokens, top_k]
  void* out;                // [tokens, n] bf16 bits or f32
  int out_f32;
  int n, k, tokens, top_k;
  int tiles;                // row tiles per token; the grid is tiles * tokens blocks
  int xcd_group;            // row tiles an XCD takes for one token before it turns to the next token (see the kernel)
};

// What a down block of the one-launch chain (gemv_chain.hpp) waits for: its slot's readiness word reaching `need`
// (the gate/up blocks that serve a slot). The wait is bounded: after `spins` polls the wavefront reports through
// `status` and goes on with whatever the row holds, so every wavefront of the grid exits.
struct SlotAwait {
  unsigned* ready;
  int stride;
  unsigned need;
  unsigned wrap;
  unsigned spins;
  int* status;
};
// A word above `wrap` was never zeroed by its owner: not ready, and the wait will run out.
__device__ __forceinline__ bool slot_ready_now(const unsigned* word, unsigned need, unsigned wrap) {
  const unsigned v = static_cast<unsigned>(
      __builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))));
  return v >= need && v <= wrap;
}
__device__ __forceinline__ bool slot_wait(const unsigned* word, unsigned need, unsigned wrap, unsigned spins) {
  for (unsigned i = 0; i < spins; ++i) {
    if (slot_ready_now(word, need, wrap)) return true;
    __builtin_amdgcn_s_sleep(16);
  }
  return false;
}
// stage_issue over a row other XCDs have just written: agent-scope loads (they pass this XCD's L2), 8 bytes each.
template <int FMT, int XV>
__device__ __forceinline__ void stage_issue_agent(const uint16_t* __restrict__ x, int k, int tid, int threads, StageRegs<XV>& r) {
  const int vecs = k / 8;
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    const int v = tid + i * threads;
    const unsigned long long* src = reinterpret_cast<const unsigned long long*>(x + static_cast<size_t>(v < vecs ? v : 0) * 8);
    const unsigned long long lo = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long hi = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    r.v[i] = make_uint4(static_cast<unsigned>(lo), static_cast<unsigned>(lo >> 32), static_cast<unsigned>(hi),
                        static_cast<unsigned>(hi >> 32));
  }
}

// The body of token_down_accum_kernel for block `b` of its grid. CHAIN: the act rows come from gate/up blocks of the
// same launch (`aw`); wavefronts beyond top_k (a block sized for the gate/up part) only join the barrier.
template <int FMT, int NB, bool SPLIT, bool CHAIN>
__device__ __forceinline__ void token_down_body(const TokenDownArgs& a, const RowGeom& g, int steps, uint4* __restrict__ lds,
                                                int b, const SlotAwait* aw = nullptr) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  // Block -> (row tile, token). Consecutive blocks go to the chip's eight XCDs in turn (block b runs on XCD b % 8 as
  // the b / 8-th block there) and each XCD has an L2 of its own. An XCD therefore takes `xcd_group` of its row tiles
  // for one token, then the SAME tiles for the next token, and so on through the batch before it moves on: tokens that
  // routed to the same expert find its rows in that L2 instead of fetching them again over the fabric. A large group
  // (all of an XCD's tiles) is plain token-major order: the longest sequential walk through each expert's rows, the
  // better order while few tokens share experts.
  int t, tile;
  {
    const int G = a.xcd_group;
    if (G > 0) {     // tiles is a multiple of 8 * G
      const int seq = b >> 3;
      const int gi = seq % G, rest = seq / G;
      t = rest % a.tokens;
      tile = ((rest / a.tokens) * G + gi) * 8 + (b & 7);
    } else {
      t = b / a.tiles;
      tile = b - t * a.tiles;
    }
  }
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  const int row_vecs = kPieces * chunks;
  const int rpw = kWave >> g.l2;
  const int rows_per_block = rpw * steps;
  const int tile_row0 = tile * rows_per_block;
  float* part = reinterpret_cast<float*>(lds + a.top_k * row_vecs);   // [top_k][rows_per_block]
  if (!CHAIN || wave < a.top_k) {
    uint4* my_x = lds + wave * row_vecs;
    const float* gd = nullptr;
    const MatRef md = mat_of_view<FMT>(a.views[a.ids[static_cast<size_t>(t) * a.top_k + wave] * 3 + 2], &gd);
    // This wavefront's activation row, in the core's [piece][chunk] order. Fast set-up (a row of at most 1024
    // aligned elements): activation loads, then the first step's weight loads, then the LDS commit.
    const uint16_t* x = a.act + (static_cast<size_t>(t) * (a.top_k + 1) + wave) * a.act_stride;
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    constexpr int XV = kSplitStageVecs;
    const auto lr = lane_row<FMT, true>(md, tile_row0, a.n, a.k, g.l2);
    ChunkRegs first[NB];
    if constexpr (CHAIN) {
      // The slot's row is complete once every gate/up block that serves it has counted itself in. Ready at the first
      // look (the common case: gate/up blocks precede the down blocks in the grid): row first, then weights, as
      // below. Otherwise the first weight loads go out before the wait.
      static_assert(SPLIT, "the chain form stages a wavefront's row from registers");
      unsigned* word = aw->ready + (static_cast<size_t>(t) * a.top_k + wave) * aw->stride;
      StageRegs<XV> xr;
      bool ok = slot_ready_now(word, aw->need, aw->wrap);
      if (ok) {
        stage_issue_agent<FMT, XV>(x, a.k, lane, kWave, xr);
        issue_pass<FMT, NB>(lr, 0, g.l2, md.cs, first);
      } else {
        issue_pass<FMT, NB>(lr, 0, g.l2, md.cs, first);
        ok = slot_wait(word, aw->need, aw->wrap, aw->spins);
        stage_issue_agent<FMT, XV>(x, a.k, lane, kWave, xr);
      }
      if (lane == 0) {
        atomicInc(word, aw->wrap);                 // this reader is through: the last one returns the word to zero
        if (!ok) *aw->status = 1;
      }
      stage_commit<FMT, XV>(xr, a.k, lane, kWave, my_x);
    } else if constexpr (SPLIT) {
      StageRegs<XV> xr;
      stage_issue<FMT, XV>(x, a.k, lane, kWave, xr);
      issue_pass<FMT, NB>(lr, 0, g.l2, md.cs, first);
      stage_commit<FMT, XV>(xr, a.k, lane, kWave, my_x);
    } else {
      for (int v = lane; v < row_vecs; v += kWave) {
        const int c = v / kPieces, q = v - c * kPieces;
        my_x[q * chunks + c] = load_vec8(x, v, aligned);
      }
    }
    // The staged row is this wavefront's own: LDS keeps a wavefront's writes and reads in order, no block barrier.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float dd = load_divisor<FMT>(gd);
    int s = 0;
    if constexpr (SPLIT) {
      float acc[1];
      row_dots_pre<FMT, 1, NB>(lr, g, md.cs, my_x, chunks, 1, first, acc);   // tile_row0 < n: the grid covers n
      if (lr.li == 0) part[wave * rows_per_block + (lane >> g.l2)] = finish_dot<FMT>(acc[0], dd);
      s = 1;
    }
    for (; s < steps; ++s) {
      const int row0 = tile_row0 + s * rpw;
      if (row0 >= a.n) break;
      const auto l2 = lane_row<FMT, true>(md, row0, a.n, a.k, g.l2);
      float acc[1];
      row_dots<FMT, 1, NB>(l2, g, md.cs, my_x, chunks, 1, acc);
      if (l2.li == 0) part[wave * rows_per_block + s * rpw + (lane >> g.l2)] = finish_dot<FMT>(acc[0], dd);
    }
  }
  __syncthreads();
  for (int r = threadIdx.x; r < rows_per_block; r += blockDim.x) {
    const int row = tile_row0 + r;
    if (row >= a.n) break;
    float v = 0.f;
    for (int j = 0; j < a.top_k; ++j)
      v = fmaf(a.weights[static_cast<size_t>(t) * a.top_k + j], part[j * rows_per_block + r], v);
    const size_t at = static_cast<size_t>(t) * a.n + row;
    if (a.out_f32)
      static_cast<float*>(a.out)[at] = v;
    else
      static_cast<uint16_t*>(a.out)[at] = f32_to_bf16(v);
  }
}

// The token-major down + accumulation block with FOUR wavefronts, each carrying two routed slots of the token (j and
// j + 4): the form a launch takes whose blocks must match the gate/up blocks' size and register budget (the one-launch
// chain). A wavefront keeps two row passes in flight - its two slots' - where the eight-wavefront block relies on
// twice the wavefronts per SIMD. Per (row, slot) the chain is row_dots', the fold the same: the same bits.
// top_k <= 8, rows of at most 1024 aligned elements. CHAIN as in token_down_body.
template <int FMT, int NB, bool CHAIN>
__device__ __forceinline__ void token_down_pair_body(const TokenDownArgs& a, const RowGeom& g, int steps, uint4* __restrict__ lds,
                                                     int b, const SlotAwait* aw = nullptr) {
  constexpr int kPieces = FmtTraits<FMT>::kPieces;
  constexpr int XV = kSplitStageVecs;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  int t, tile;
  {
    const int G = a.xcd_group;
    if (G > 0) {     // tiles is a multiple of 8 * G (see token_down_body)
      const int seq = b >> 3;
      const int gi = seq % G, rest = seq / G;
      t = rest % a.tokens;
      tile = ((rest / a.tokens) * G + gi) * 8 + (b & 7);
    } else {
      t = b / a.tiles;
      tile = b - t * a.tiles;
    }
  }
  const int chunks = a.k / FmtTraits<FMT>::kElemsPerChunk;
  const int row_vecs = kPieces * chunks;
  const int rpw = kWave >> g.l2;
  const int rows_per_block = rpw * steps;
  const int tile_row0 = tile * rows_per_block;
  float* part = reinterpret_cast<float*>(lds + a.top_k * row_vecs);   // [top_k][rows_per_block]
  const int j0 = wave, j1 = wave + kWavesPerBlock;
  if (j0 < a.top_k) {
    const bool two = j1 < a.top_k;
    const int jb = two ? j1 : j0;
    const size_t r0 = static_cast<size_t>(t) * a.top_k + j0, r1 = static_cast<size_t>(t) * a.top_k + jb;
    // wave-uniform by construction: saying so keeps the table entries in scalar registers
    const int e0 = __builtin_amdgcn_readfirstlane(a.ids[r0]), e1 = __builtin_amdgcn_readfirstlane(a.ids[r1]);
    unsigned v0 = 0, v1 = 0;
    unsigned *w0 = nullptr, *w1 = nullptr;
    if constexpr (CHAIN) {
      // The readiness words are asked for before the table entries: their trip to the memory side runs beside the
      // ids -> entry -> address chain.
      w0 = aw->ready + r0 * aw->stride;
      w1 = aw->ready + r1 * aw->stride;
      v0 = __hip_atomic_load(w0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v1 = __hip_atomic_load(w1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const float *gd0 = nullptr, *gd1 = nullptr;
    const MatRef m0 = mat_of_view<FMT>(a.views[e0 * 3 + 2], &gd0);
    const MatRef m1 = mat_of_view<FMT>(a.views[e1 * 3 + 2], &gd1);
    const uint16_t* x0 = a.act + (static_cast<size_t>(t) * (a.top_k + 1) + j0) * a.act_stride;
    const uint16_t* x1 = a.act + (static_cast<size_t>(t) * (a.top_k + 1) + jb) * a.act_stride;
    uint4* my0 = lds + j0 * row_vecs;
    uint4* my1 = lds + jb * row_vecs;
    auto lr0 = lane_row<FMT, true>(m0, tile_row0, a.n, a.k, g.l2);
    auto lr1 = lane_row<FMT, true>(m1, tile_row0, a.n, a.k, g.l2);
    ChunkRegs f0[NB], f1[NB];
    StageRegs<XV> xa, xb;
    if constexpr (CHAIN) {
      auto ready = [&](unsigned v) {
        const unsigned u = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
        return u >= aw->need && u <= aw->wrap;
      };
      // The first weight passes go out before the rows are looked for: they travel while the wavefront waits.
      issue_pass<FMT, NB>(lr0, 0, g.l2, m0.cs, f0);
      if (two) issue_pass<FMT, NB>(lr1, 0, g.l2, m1.cs, f1);
      bool ok = ready(v0) && (!two || ready(v1));
      if (!ok) {
        ok = slot_wait(w0, aw->need, aw->wrap, aw->spins);
        if (two) ok = slot_wait(w1, aw->need, aw->wrap, aw->spins) && ok;
      }
      stage_issue_agent<FMT, XV>(x0, a.k, lane, kWave, xa);
      if (two) stage_issue_agent<FMT, XV>(x1, a.k, lane, kWave, xb);
      if (lane == 0) {
        atomicInc(w0, aw->wrap);                   // this reader is through: the last one returns the word to zero
        if (two) atomicInc(w1, aw->wrap);
        if (!ok) *aw->status = 1;
      }
    } else {
      stage_issue<FMT, XV>(x0, a.k, lane, kWave, xa);
      if (two) stage_issue<FMT, XV>(x1, a.k, lane, kWave, xb);
      issue_pass<FMT, NB>(lr0, 0, g.l2, m0.cs, f0);
      if (two) issue_pass<FMT, NB>(lr1, 0, g.l2, m1.cs, f1);
    }
    stage_commit<FMT, XV>(xa, a.k, lane, kWave, my0);
    if (two) stage_commit<FMT, XV>(xb, a.k, lane, kWave, my1);
    // The staged rows are this wavefront's own: LDS keeps a wavefront's writes and reads in order, no block barrier.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float dd0 = load_divisor<FMT>(gd0), dd1 = load_divisor<FMT>(gd1);
    for (int s = 0; s < steps; ++s) {
      const int row0 = tile_row0 + s * rpw;
      if (row0 >= a.n) break;
      const bool more = s + 1 < steps && row0 + rpw < a.n;
      const int at = s * rpw + (lane >> g.l2);
      float acc[1];
      row_dots_pre<FMT, 1, NB>(lr0, g, m0.cs, my0, chunks, 1, f0, acc);
      if (lr0.li == 0) part[j0 * rows_per_block + at] = finish_dot<FMT>(acc[0], dd0);
      if (more) {   // this slot's next row group goes out while the other slot's current one is consumed
        lr0 = lane_row<FMT, true>(m0, row0 + rpw, a.n, a.k, g.l2);
        issue_pass<FMT, NB>(lr0, 0, g.l2, m0.cs, f0);
      }
      if (two) {
        row_dots_pre<FMT, 1, NB>(lr1, g, m1.cs, my1, chunks, 1, f1, acc);
        if (lr1.li == 0) part[j1 * rows_per_block + at] = finish_dot<FMT>(acc[0], dd1);
        if (more) {
          lr1 = lane_row<FMT, true>(m1, row0 + rpw, a.n, a.k, g.l2);
          issue_pass<FMT, NB>(lr1, 0, g.l2, m1.cs, f1);
        }
      }
    }
  }
  __syncthreads();
  for (int r = threadIdx.x; r < rows_per_block; r += blockDim.x) {
    const int row = tile_row0 + r;
    if (row >= a.n) break;
    float v = 0.f;
    for (int j = 0; j < a.top_k; ++j)
      v = fmaf(a.weights[static_cast<size_t>(t) * a.top_k + j], part[j * rows_per_block + r], v);
    const size_t at = static_cast<size_t>(t) * a.n + row;
    if (a.out_f32)
      static_cast<float*>(a.out)[at] = v;
    else
      static_cast<uint16_t*>(a.out)[at] = f32_to_bf16(v);
  }
}

template <int FMT, int NB, bool SPLIT>
__global__ __launch_bounds__(1024) void token_down_accum_kernel(TokenDownArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  token_down_body<FMT, NB, SPLIT, false>(a, g, steps, lds, static_cast<int>(blockIdx.x));
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
  const int32_t* act_rows;  // matrix-core form only, nullable: activation row of each segment row
  int once;                 // every segment fits one pass over its expert (nontemporal loads)
  int gate_up;              // matrix-core form only, `which` unused, bf16 out: 1 = gate and up rows + SwiGLU in one
                            // launch; 2 = gate rows to `out`, up rows to `out_up`
  float limit;              // the SwiGLU clamp of form 1
  void* out_up;             // form 2
  // matrix-core form, NVFP4 experts: the activations are NVFP4 rows (act = codes, act_stride = bytes per row)
  const uint8_t* a4_scales = nullptr;   // e4m3 [rows, a4_scale_stride]
  size_t a4_scale_stride = 0;
  const float* a4_gs = nullptr;         // [rows]
};

template <int FMT, int NB, bool NT>
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
      const auto lr = lane_row<FMT, NT>(mat, row0, a.n, a.k, g.l2);
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

}  // namespace dgpp_amd

#include "gemv_mfma_kernels.hpp"

namespace dgpp_amd {

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
// `count` problems (<= kMaxDenseProblems) of one k, one row count (<= the rows one stage holds) in one vector-core launch.
hipError_t launch_dense_multi(int fmt, const DenseArgs* problems, int count, hipStream_t stream);
template <int FMT> hipError_t launch_dense_multi_fmt(const DenseArgs* problems, int count, hipStream_t stream);
hipError_t launch_slot_gate_up(int fmt, const SlotArgs& a, hipStream_t stream);
hipError_t launch_select_gate_up(int fmt, const SlotArgs& a, const SelectArgs& sel, hipStream_t stream);
hipError_t launch_slot_down(int fmt, const SlotArgs& a, hipStream_t stream);
hipError_t launch_grouped(int fmt, const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream);

// Routed gate/up + SwiGLU with the two projections in different formats (one block-FP8, one NVFP4).
hipError_t launch_slot_gate_up_mixed(const SlotArgs& a, int gate_fp4, hipStream_t stream);

// Token-major routed down + accumulation (vector core).
hipError_t launch_token_down(int fmt, const TokenDownArgs& a, hipStream_t stream);
template <int FMT> hipError_t launch_token_down_fmt(const TokenDownArgs& a, hipStream_t stream);

// The matrix-core launchers proper (the *_mma_* entry points).
hipError_t launch_dense_mma(int fmt, const DenseArgs& a, float* ws, size_t ws_bytes, hipStream_t stream);
// Two FP8 (F32 grid) problems of one k and m in one launch; ws as in launch_dense_mma (both problems' partials).
hipError_t launch_dense_mma_pair_fp8(const DenseArgs& a0, const DenseArgs& a1, float* ws, size_t ws_bytes, hipStream_t stream);
hipError_t launch_grouped_mma(int fmt, const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream);
template <int FMT> hipError_t launch_dense_mma_fmt(const DenseArgs& a, float* ws, size_t ws_bytes, hipStream_t stream);
template <int FMT> hipError_t launch_grouped_mma_fmt(const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream);

// ---- the routed chain in one launch (gemv_chain.hpp) -------------------------------------------------------
constexpr int kReadyStride = 32;            // words between two slots' readiness words: a 128-byte line each
constexpr unsigned kChainDefaultSpins = 1u << 18;

struct ChainArgs {
  SlotArgs gu;        // x rows, ids, views, out = act [slots, out_stride], n = inter, k = hidden
  TokenDownArgs dn;   // act rows, ids, views, weights, out, n = hidden, k = inter
  unsigned* ready;    // [tokens * top_k * kReadyStride], zero at rest
  int* status;        // one word, raised when a wait gave up
  int gu_tiles;       // gate/up row tiles per slot
  int gu_blocks;      // gu_tiles * tokens * top_k
  unsigned spins;
};

// Whether the one-launch form takes this problem (otherwise the caller runs the two launches).
inline bool slot_chain_fits(const ChainArgs& c) {
  const SlotArgs& u = c.gu;
  const TokenDownArgs& d = c.dn;
  const int K = u.top_k;
  if (K < 1 || K > 8 || d.tokens < 1 || d.tokens * K > 128) return false;
  if (tune_get(kTuneCore) == 2 || tune_get(kTuneSplitStage) == 1) return false;
  // the fast set-ups of both parts: whole rows held in registers between their loads and the LDS commit
  if (u.k > 8 * kSplitStageVecs * kBlockThreads || (u.x_stride & 7u) != 0 || (reinterpret_cast<uintptr_t>(u.x) & 15u) != 0) return false;
  if (d.k > 8 * kSplitStageVecs * kWave || (d.act_stride & 7u) != 0 || (reinterpret_cast<uintptr_t>(d.act) & 15u) != 0) return false;
  return true;
}

// The pass widths the chain kernel is compiled for (a lane's loads in flight per row and pass: 1, 2 or 4).
template <int FMT>
inline bool slot_chain_widths_ok(int k_gate_up, int k_down) {
  const int a = geom_for<FMT>(k_gate_up).nb, b = geom_for<FMT>(k_down).nb;
  auto ok = [](int nb) { return nb == 1 || nb == 2 || nb == 4; };
  return ok(a) && ok(b);
}

// `sel` non-null: one token, the selection repeated by every block (select_chain_kernel).
hipError_t launch_slot_chain(int fmt, const ChainArgs& c, const SelectArgs* sel, hipStream_t stream);
template <int FMT> hipError_t launch_slot_chain_fmt(const ChainArgs& c, const SelectArgs* sel, hipStream_t stream);

// Per-format implementations.
template <int FMT> hipError_t launch_dense_fmt(const DenseArgs& a, hipStream_t stream);
template <int FMT> hipError_t launch_slot_gate_up_fmt(const SlotArgs& a, hipStream_t stream);
template <int FMT> hipError_t launch_select_gate_up_fmt(const SlotArgs& a, const SelectArgs& sel, hipStream_t stream);
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

// Whether the dense matrix-core launch runs its K parts in separate blocks through a workspace when it is given one
// that is large enough (launch_dense_mfma's rule): more than one part, and row tiles that leave the chip under-filled.
inline bool dense_mfma_would_split(int parts, int m, int n) {
  return parts > 1 && static_cast<size_t>((n + 63) / 64) * static_cast<size_t>((m + 15) / 16) < 1024;
}

// Row groups per block of the dense matrix-core launch that runs the four parts of K side by side inside a block
// (0: the row-tile form). Four up to one round of the chip's 256 CUs - one such block fills a CU, and 272 tiles, two
// rounds with the second nearly empty, measured slower than the row-tile form; two (blocks half the size, two to a CU)
// for up to eight activation rows when the row tiles just exceed a round. Bench switch 11: 1 never, 2 four, 3 two.
constexpr size_t kTeamsMaxTiles = 256;
constexpr size_t kTeamsMaxTilesHalf = 320;
inline int dense_mfma_team_row_groups(int parts, int m, int n, bool plain) {
  const int knob = tune_get(kTuneTeams);
  if (!plain || parts != 4 || knob == 1) return 0;
  const size_t tiles = static_cast<size_t>((n + 63) / 64) * static_cast<size_t>((m + 15) / 16);
  if (knob == 2 || tiles <= kTeamsMaxTiles) return 4;
  if ((knob == 3 || tiles <= kTeamsMaxTilesHalf) && m <= 8) return 2;
  return 0;
}

// The bodies, included by the per-format translation units.
#ifdef DGPP_GEMV_IMPL
template <class F>
inline void dispatch_bool(bool v, F&& f) {
  if (v) f(std::true_type{});
  else f(std::false_type{});
}

// The GEMV launchers run the vector ALU core (fastest while one or two activation rows ride on a weight
// pass); the bench switch moves them to the matrix-core form, which the *_mma_* launchers always use.
inline bool use_mfma_core() { return tune_get(kTuneCore) == 2; }

// `ws` (nullable) holds parts * m * n floats: the K parts then run in separate blocks and a second
// launch folds them (same bits); worth it only when the unsplit grid leaves the chip under-filled.

template <int FMT>
hipError_t launch_dense_mfma(const DenseArgs& a, hipStream_t stream, float* ws, size_t ws_bytes) {
  const MGeom g = mgeom<FMT>(a.k);
  const unsigned gx = static_cast<unsigned>((a.n + 63) / 64), gy = static_cast<unsigned>((a.m + kTileCols - 1) / kTileCols);
  const size_t need = static_cast<size_t>(g.parts) * a.m * a.n * sizeof(float);
  const bool split = ws != nullptr && ws_bytes >= need && dense_mfma_would_split(g.parts, a.m, a.n) && a.a4_scales == nullptr;
  const dim3 grid(gx, gy, split ? g.parts : 1);
  hipError_t err = hipSuccess;
  // Without a workspace the four parts of K run side by side inside a block while the row tiles alone would leave
  // most SIMDs one wavefront.
  const int rg = dense_mfma_team_row_groups(g.parts, a.m, a.n, !split && a.act_up == nullptr && a.a4_scales == nullptr);
  if (rg != 0) {
    dispatch_bool(a.once != 0, [&](auto ntc) {
      auto launch = [&](auto rgc) {
        constexpr int RG = decltype(rgc)::value;
        auto kern = mfma_dense_teams_kernel<FMT, kMfmaNB, decltype(ntc)::value, RG>;
        constexpr size_t lds = TeamShape<RG>::kLdsUnits * sizeof(uint4);
        err = ensure_lds(kern, lds);
        const unsigned bx = static_cast<unsigned>((a.n + RG * kGroupRows - 1) / (RG * kGroupRows));
        if (err == hipSuccess) hipLaunchKernelGGL(kern, dim3(bx, gy), dim3(TeamShape<RG>::kThreads), lds, stream, a, g);
      };
      if (rg == 4) launch(std::integral_constant<int, 4>{});
      else launch(std::integral_constant<int, 2>{});
    });
    return err != hipSuccess ? err : hipGetLastError();
  }
  dispatch_bool(a.once != 0, [&](auto ntc) {
    auto go = [&](auto kern) {
      constexpr size_t lds = kBlockMfmaLdsUnits * sizeof(uint4);
      err = ensure_lds(kern, lds);
      if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g, split ? ws : nullptr);
    };
    if constexpr (FMT == kFmtFp8F32) {   // the SwiGLU-staging form exists for the reference's one launcher of it
      if (a.act_up) return go(mfma_dense_kernel<FMT, kMfmaNB, decltype(ntc)::value, true>);
    }
    if constexpr (FMT == kFmtNvfp4) {    // the activation-quantized form (never split: its epilogue is its own)
      if (a.a4_scales) return go(mfma_dense_kernel<FMT, kMfmaNB, decltype(ntc)::value, false, true>);
    }
    go(mfma_dense_kernel<FMT, kMfmaNB, decltype(ntc)::value, false>);
  });
  if (err != hipSuccess) return err;
  if (split) {
    const int64_t total = static_cast<int64_t>(a.m) * a.n;
    hipLaunchKernelGGL(fold_parts_kernel<FMT>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream, ws,
                       g.parts, a.m, a.n, a.global, a.out, a.out_f32, a.out_stride);
  }
  return hipGetLastError();
}

#ifdef DGPP_GEMV_PAIR
hipError_t launch_dense_mma_pair_fp8(const DenseArgs& a0, const DenseArgs& a1, float* ws, size_t ws_bytes, hipStream_t stream) {
  constexpr int FMT = kFmtFp8F32;
  const MGeom g = mgeom<FMT>(a0.k);
  const unsigned t0 = static_cast<unsigned>((a0.n + 63) / 64), t1 = static_cast<unsigned>((a1.n + 63) / 64);
  const unsigned gy = static_cast<unsigned>((a0.m + kTileCols - 1) / kTileCols);
  const size_t need = static_cast<size_t>(g.parts) * a0.m * (static_cast<size_t>(a0.n) + a1.n) * sizeof(float);
  const bool split = ws != nullptr && g.parts > 1 && ws_bytes >= need && static_cast<size_t>(t0 + t1) * gy < 1024;
  const dim3 grid(t0 + t1, gy, split ? g.parts : 1);
  hipError_t err = hipSuccess;
  dispatch_bool(a0.once != 0, [&](auto ntc) {
    auto kern = mfma_dense_pair_kernel<FMT, kMfmaNB, decltype(ntc)::value>;
    constexpr size_t lds = kBlockMfmaLdsUnits * sizeof(uint4);
    err = ensure_lds(kern, lds);
    if (err == hipSuccess)
      hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a0, a1, static_cast<int>(t0), g, split ? ws : nullptr);
  });
  if (err != hipSuccess) return err;
  if (split) {
    const DenseArgs* both[2] = {&a0, &a1};
    float* at = ws;
    for (const DenseArgs* a : both) {
      const int64_t total = static_cast<int64_t>(a->m) * a->n;
      hipLaunchKernelGGL(fold_parts_kernel<FMT>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream, at,
                         g.parts, a->m, a->n, a->global, a->out, a->out_f32, a->out_stride);
      at += static_cast<size_t>(g.parts) * a->m * a->n;
    }
  }
  return hipGetLastError();
}
#endif

template <int FMT>
hipError_t launch_grouped_mfma(const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream) {
  const MGeom g = mgeom<FMT>(a.k);
  const dim3 grid(static_cast<unsigned>((a.n + 63) / 64), static_cast<unsigned>(n_segs), static_cast<unsigned>(z_ext));
  hipError_t err = hipSuccess;
  if constexpr (FMT == kFmtNvfp4) {
    if (a.a4_scales != nullptr) {   // the activation-quantized form
      dispatch_bool(a.once != 0, [&](auto ntc) {
        auto kern = mfma_grouped_kernel<FMT, kMfmaNB, decltype(ntc)::value, false, true>;
        constexpr size_t lds = kBlockMfmaLdsUnits * sizeof(uint4);
        err = ensure_lds(kern, lds);
        if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g);
      });
      return err != hipSuccess ? err : hipGetLastError();
    }
  }
  // gate + up in one launch: while the grid is small (a few rounds of the chip) a block's wavefronts split into gate
  // walkers and up walkers - twice the blocks, half the walk each (C4 100 -> 90 us); a large grid keeps every wavefront
  // on both walks (C5: 1100 us against 1140 us split).
  // (bench / test switch 14: 1 never splits, 2 always)
  const int walks = tune_get(kTuneGateUpWalks);
  const bool split_walks = a.gate_up != 0 && walks != 1 && (walks == 2 || static_cast<size_t>(grid.x) * grid.y * grid.z <= 2048);
  dispatch_bool(a.once != 0, [&](auto ntc) {
    dispatch_bool(a.gate_up != 0, [&](auto guc) {
      dispatch_bool(split_walks, [&](auto swc) {
        constexpr bool GU = decltype(guc)::value, GUW = decltype(swc)::value;
        if constexpr (GUW && !GU) {
          err = hipErrorInvalidValue;   // not reached: split_walks implies gate_up
        } else {
          auto kern = mfma_grouped_kernel<FMT, kMfmaNB, decltype(ntc)::value, GU, false, GUW>;
          constexpr size_t lds = kBlockMfmaLdsUnits * sizeof(uint4);
          const dim3 gu_grid(static_cast<unsigned>((a.n + 31) / 32), grid.y, grid.z);
          err = ensure_lds(kern, lds);
          if (err == hipSuccess) hipLaunchKernelGGL(kern, GUW ? gu_grid : grid, dim3(kBlockThreads), lds, stream, a, g);
        }
      });
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}

// Slots per run in the matrix-core slot kernels: bounded by the LDS of the per-wavefront stages.
template <int FMT>
inline int mfma_run_cap(const SlotArgs& a, const MGeom& g, int max_run) {
  if (a.order == nullptr && !a.match) return 1;
  const int tuned = tune_get(kTuneSlotRun);
  int cap = tuned > 0 && tuned < max_run ? tuned : max_run;
  while (cap > 1 && (kWavesPerBlock * slot_wave_units<FMT>(cap, g) + kSlotRedUnits) * sizeof(uint4) > 48 * 1024) --cap;
  return cap;
}
template <int FMT>
inline size_t mfma_slot_lds(int maxm, const MGeom& g) {
  return (static_cast<size_t>(kWavesPerBlock) * slot_wave_units<FMT>(maxm, g) + kSlotRedUnits) * sizeof(uint4);
}

template <int FMT>
hipError_t launch_slot_gate_up_mfma(const SlotArgs& a, hipStream_t stream) {
  const MGeom g = mgeom<FMT>(a.k);
  const int rows_per_block = kWavesPerBlock / g.parts * kGroupRows;
  const dim3 grid(static_cast<unsigned>((a.n + rows_per_block - 1) / rows_per_block), static_cast<unsigned>(a.slots));
  const int cap = mfma_run_cap<FMT>(a, g, 2);
  hipError_t err = hipSuccess;
  auto go = [&](auto mc) {
    constexpr int MAXM = decltype(mc)::value;
    auto kern = slot_gate_up_mfma_kernel<FMT, kMfmaNB, MAXM>;
    const size_t lds = mfma_slot_lds<FMT>(MAXM, g);
    err = ensure_lds(kern, lds);
    if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g);
  };
  if (cap >= 2) go(std::integral_constant<int, 2>{});
  else go(std::integral_constant<int, 1>{});
  return err != hipSuccess ? err : hipGetLastError();
}

template <int FMT>
hipError_t launch_slot_down_mfma(const SlotArgs& a, hipStream_t stream) {
  const MGeom g = mgeom<FMT>(a.k);
  const int rows_per_block = kWavesPerBlock / g.parts * kGroupRows;
  const dim3 grid(static_cast<unsigned>((a.n + rows_per_block - 1) / rows_per_block), static_cast<unsigned>(a.slots));
  const int cap = mfma_run_cap<FMT>(a, g, 2);
  hipError_t err = hipSuccess;
  auto go = [&](auto mc) {
    constexpr int MAXM = decltype(mc)::value;
    auto kern = slot_down_mfma_kernel<FMT, kMfmaNB, MAXM>;
    const size_t lds = mfma_slot_lds<FMT>(MAXM, g);
    err = ensure_lds(kern, lds);
    if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g);
  };
  if (cap >= 2) go(std::integral_constant<int, 2>{});
  else go(std::integral_constant<int, 1>{});
  return err != hipSuccess ? err : hipGetLastError();
}

template <int FMT>
hipError_t launch_dense_fmt(const DenseArgs& a, hipStream_t stream) {
  if (use_mfma_core()) return launch_dense_mfma<FMT>(a, stream, nullptr, 0);
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long block_steps = (a.n + rows_per_step - 1) / rows_per_step;
  int steps = pick_steps(block_steps);
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  const dim3 grid(static_cast<unsigned>((block_steps + steps - 1) / steps));
  const size_t lds = stage_bytes(a.m, a.k);
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    auto go = [&](auto rc) {
      constexpr int MAXR = decltype(rc)::value;
      dispatch_bool(a.once != 0, [&](auto ntc) {
        auto kern = gemv_dense_kernel<FMT, MAXR, NB, decltype(ntc)::value>;
        err = ensure_lds(kern, lds);
        if (err != hipSuccess) return;
        hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g, steps);
      });
    };
    if (a.m == 1) go(std::integral_constant<int, 1>{});
    else if (a.m == 2) go(std::integral_constant<int, 2>{});
    else if (a.m <= 4) go(std::integral_constant<int, 4>{});
    else go(std::integral_constant<int, 8>{});
  });
  return err != hipSuccess ? err : hipGetLastError();
}

template <int FMT>
hipError_t launch_dense_multi_fmt(const DenseArgs* problems, int count, hipStream_t stream) {
  const DenseArgs& first = problems[0];
  const RowGeom g = geom_for<FMT>(first.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  long long all_steps = 0;
  for (int i = 0; i < count; ++i) all_steps += (problems[i].n + rows_per_step - 1) / rows_per_step;
  int steps = pick_steps(all_steps);
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  DenseMultiArgs ma{};
  ma.count = count;
  long long end = 0;
  for (int i = 0; i < count; ++i) {
    ma.p[i] = problems[i];
    const long long block_steps = (problems[i].n + rows_per_step - 1) / rows_per_step;
    end += (block_steps + steps - 1) / steps;
    ma.tile_end[i] = static_cast<int>(end);
  }
  if (end > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  const dim3 grid(static_cast<unsigned>(end));
  const size_t lds = stage_bytes(first.m, first.k);
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    auto go = [&](auto rc) {
      constexpr int MAXR = decltype(rc)::value;
      auto kern = gemv_dense_multi_kernel<FMT, MAXR, NB, true>;   // every problem's weights stream through once
      err = ensure_lds(kern, lds);
      if (err != hipSuccess) return;
      hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, ma, g, steps);
    };
    if (first.m == 1) go(std::integral_constant<int, 1>{});
    else if (first.m == 2) go(std::integral_constant<int, 2>{});
    else if (first.m <= 4) go(std::integral_constant<int, 4>{});
    else go(std::integral_constant<int, 8>{});
  });
  return err != hipSuccess ? err : hipGetLastError();
}

// Slots of a run one block serves: a shared expert read once for up to this many slots. Bounded by the
// LDS a block may take without giving up residency (16 KB of staged activations) and by the
// accumulators a lane holds.
constexpr int kGateUpRun = 2;
constexpr int kGateUpRunBatch = 4;
constexpr int kDownRun = 4;
inline int run_cap_for(const SlotArgs& a, int max_run) {
  if (a.order == nullptr && !a.match) return 1;   // slots in layout order and no way to find the sharers
  const int tuned = tune_get(kTuneSlotRun);
  int cap = tuned > 0 ? tuned : max_run;
  // 32 KB of staged rows keeps five blocks on a CU; two slots per weight pass also halve the decode work per slot
  while (cap > 1 && (cap > max_run || stage_bytes(cap, a.k) > 32 * 1024)) --cap;
  return cap;
}

template <int FMT>
hipError_t launch_slot_gate_up_fmt(const SlotArgs& a, hipStream_t stream) {
  if (use_mfma_core()) return launch_slot_gate_up_mfma<FMT>(a, stream);
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long per_slot = (a.n + rows_per_step - 1) / rows_per_step;
  int steps = pick_steps(per_slot * a.slots);
  if (a.once && a.slots > a.top_k + 1) steps = 2;   // a decode batch of 2 - 8 tokens: measured best (one token: 1)
  if (a.want_shared && a.once) steps = 1;           // one expert's rows over few runs: as many blocks as there are row groups
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  const dim3 grid(static_cast<unsigned>((per_slot + steps - 1) / steps), static_cast<unsigned>(a.slots));
  // Larger batches (many slots per expert, an order given): runs of four where the rows fit the stage.
  const int cap = run_cap_for(a, (!a.once && a.order != nullptr) ? kGateUpRunBatch : kGateUpRun);
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    const bool split = tune_get(kTuneSplitStage) != 1 && a.k <= 8 * kSplitStageVecs * kBlockThreads &&
                       (a.x_stride & 7u) == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0;
    // Nontemporal loads only with the split set-up (the decode form); shared slots are read by every token.
    const bool nt = split && a.once && !a.want_shared;
    auto go = [&](auto mc, auto sc, auto ntc) {
      constexpr int MAXM = decltype(mc)::value;
      auto kern = slot_gate_up_kernel<FMT, NB, MAXM, decltype(sc)::value, decltype(ntc)::value>;
      err = ensure_lds(kern, stage_bytes(MAXM, a.k));   // one staged row of a wide k can exceed the default LDS ceiling
      if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), stage_bytes(MAXM, a.k), stream, a, g, steps);
    };
    auto go_m = [&](auto mc) {
      if (nt) go(mc, std::true_type{}, std::true_type{});
      else if (split) go(mc, std::true_type{}, std::false_type{});
      else go(mc, std::false_type{}, std::false_type{});
    };
    if constexpr (NB <= 4) {   // two accumulators per slot and matrix: four slots fit the registers up to four loads per pass
      if (cap >= kGateUpRunBatch) return go(std::integral_constant<int, kGateUpRunBatch>{}, std::false_type{}, std::false_type{});
    }
    if (cap >= kGateUpRun) go_m(std::integral_constant<int, kGateUpRun>{});
    else go_m(std::integral_constant<int, 1>{});
  });
  return err != hipSuccess ? err : hipGetLastError();
}

// The mixed-format gate/up launch (routed slots only; one slot per block - the form is rare enough to go without runs).
#ifdef DGPP_GEMV_MIXED
hipError_t launch_slot_gate_up_mixed(const SlotArgs& a, int gate_fp4, hipStream_t stream) {
  const RowGeom g8 = geom_for<kFmtFp8F32>(a.k), g4 = geom_for<kFmtNvfp4>(a.k);
  const int step8 = kWavesPerBlock * (kWave >> g8.l2), step4 = kWavesPerBlock * (kWave >> g4.l2);
  const int unit = step8 > step4 ? step8 : step4;   // both are powers of two: the larger is a multiple of the smaller
  const long long per_slot = (a.n + unit - 1) / unit;
  const int steps = pick_steps(per_slot * a.slots);
  const int rows_per_block = unit * steps;
  const dim3 grid(static_cast<unsigned>((a.n + rows_per_block - 1) / rows_per_block), static_cast<unsigned>(a.slots));
  const size_t lds = 2 * stage_bytes(1, a.k) + 2 * static_cast<size_t>(rows_per_block) * sizeof(float);
  hipError_t err = hipSuccess;
  // Loads in flight per lane and row: the largest of 4, 2, 1 that divides the lane's chunk count (the chain per row
  // does not depend on it; the full set of pass widths would square the number of kernels of this rare form).
  auto pass_width = [](const RowGeom& g) { return g.P % 4 == 0 ? 4 : (g.P % 2 == 0 ? 2 : 1); };
  dispatch_nb(pass_width(g8), [&](auto n8) {
    dispatch_nb(pass_width(g4), [&](auto n4) {
      dispatch_bool(gate_fp4 != 0, [&](auto gf) {
        constexpr int N8 = decltype(n8)::value, N4 = decltype(n4)::value;
        if constexpr (N8 > 4 || N8 == 3 || N4 > 4 || N4 == 3) {
          err = hipErrorInvalidValue;   // never taken: pass_width returns 4, 2 or 1
          return;
        } else {
        auto kern = slot_gate_up_mixed_kernel<N8, N4, decltype(gf)::value>;
        err = ensure_lds(kern, lds);
        if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g8, g4, rows_per_block);
        }
      });
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}
#endif

// The fused selection + gate/up launch; the caller has checked its limits (capi.hip, select_gate_up_fits).
template <int FMT>
hipError_t launch_select_gate_up_fmt(const SlotArgs& a, const SelectArgs& sel, hipStream_t stream) {
  const RowGeom g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long per_slot = (a.n + rows_per_step - 1) / rows_per_step;
  int steps = pick_steps(per_slot * a.slots);
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  const dim3 grid(static_cast<unsigned>((per_slot + steps - 1) / steps), static_cast<unsigned>(a.slots));
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    auto kern = select_gate_up_kernel<FMT, NB>;
    const size_t lds = stage_bytes(1, a.k) + kWave * sizeof(int32_t);
    err = ensure_lds(kern, lds);
    if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, sel, g, steps);
  });
  return err != hipSuccess ? err : hipGetLastError();
}

// Row tiles (grid x) and steps of a vector-form down launch.
// [token, tile].
template <int FMT>
inline void slot_down_grid(const SlotArgs& a, RowGeom& g, int& steps, unsigned& tiles) {
  g = geom_for<FMT>(a.k);
  const int rows_per_step = kWavesPerBlock * (kWave >> g.l2);
  const long long per_slot = (a.n + rows_per_step - 1) / rows_per_step;
  steps = pick_steps(per_slot * a.slots);
  if (a.want_shared && a.once) steps = 1;
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  tiles = static_cast<unsigned>((per_slot + steps - 1) / steps);
}

template <int FMT>
hipError_t launch_slot_down_fmt(const SlotArgs& a, hipStream_t stream) {
  if (use_mfma_core()) return launch_slot_down_mfma<FMT>(a, stream);
  RowGeom g;
  int steps;
  unsigned tiles;
  slot_down_grid<FMT>(a, g, steps, tiles);
  const dim3 grid(tiles, static_cast<unsigned>(a.slots));
  const int cap = run_cap_for(a, kDownRun);
  hipError_t err = hipSuccess;
  auto launch = [&](auto kern, int rows) {
    err = ensure_lds(kern, stage_bytes(rows, a.k));   // one staged row of a wide k can exceed the default LDS ceiling
    if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), stage_bytes(rows, a.k), stream, a, g, steps);
  };
  if (a.acc_out != nullptr) {   // a shared pass that ends with the token's accumulation: cached loads, every run length
    dispatch_nb(g.nb, [&](auto nbc) {
      constexpr int NB = decltype(nbc)::value;
      if (cap >= kDownRun) launch(slot_down_kernel<FMT, NB, kDownRun, false, true>, kDownRun);
      else if (cap >= 2) launch(slot_down_kernel<FMT, NB, 2, false, true>, 2);
      else launch(slot_down_kernel<FMT, NB, 1, false, true>, 1);
    });
    return err != hipSuccess ? err : hipGetLastError();
  }
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    dispatch_bool(a.once && !a.want_shared, [&](auto ntc) {
      constexpr bool NT = decltype(ntc)::value;
      if (cap >= kDownRun) launch(slot_down_kernel<FMT, NB, kDownRun, NT>, kDownRun);
      else if (cap >= 2) launch(slot_down_kernel<FMT, NB, 2, NT>, 2);
      else launch(slot_down_kernel<FMT, NB, 1, NT>, 1);
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}

template <int FMT>
hipError_t launch_token_down_fmt(const TokenDownArgs& a, hipStream_t stream) {
  const RowGeom g = geom_for<FMT>(a.k);
  const int rpw = kWave >> g.l2;
  const long long wave_steps = static_cast<long long>((a.n + rpw - 1) / rpw) * a.tokens * a.top_k;
  int steps = static_cast<int>(wave_steps / 16384);
  steps = steps < 2 ? 2 : (steps > 8 ? 8 : steps);   // two row groups per wavefront measured best from one token on
  if (tune_get(kTuneSlotSteps) > 0) steps = tune_get(kTuneSlotSteps);
  const int rows_per_block = rpw * steps;
  TokenDownArgs b = a;
  b.tiles = (a.n + rows_per_block - 1) / rows_per_block;
  // Tokens share experts often enough to pay for the XCD-local order from about a quarter of the experts in use.
  b.xcd_group = 0;
  {
    int want = tune_get(kTuneXcdGroup) > 0 ? tune_get(kTuneXcdGroup) : (a.tokens * a.top_k * 4 >= 256 ? 1 : 0);
    if (a.tokens > 1 && want > 0 && b.tiles % (8 * want) == 0) b.xcd_group = want;
  }
  if (static_cast<long long>(b.tiles) * a.tokens > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  const dim3 grid(static_cast<unsigned>(b.tiles) * static_cast<unsigned>(a.tokens));
  const size_t lds = static_cast<size_t>(a.top_k) * (stage_bytes(1, a.k) + static_cast<size_t>(rows_per_block) * sizeof(float));
  hipError_t err = hipSuccess;
  dispatch_nb(g.nb, [&](auto nbc) {
    constexpr int NB = decltype(nbc)::value;
    const bool split = tune_get(kTuneSplitStage) != 1 && a.k <= 8 * kSplitStageVecs * kWave && (a.act_stride & 7u) == 0 &&
                       (reinterpret_cast<uintptr_t>(a.act) & 15u) == 0;
    auto go = [&](auto kern) {
      err = ensure_lds(kern, lds);
      if (err == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(a.top_k * kWave), lds, stream, b, g, steps);
    };
    if (split) go(token_down_accum_kernel<FMT, NB, true>);
    else go(token_down_accum_kernel<FMT, NB, false>);
  });
  return err != hipSuccess ? err : hipGetLastError();
}

template <int FMT>
hipError_t launch_dense_mma_fmt(const DenseArgs& a, float* ws, size_t ws_bytes, hipStream_t stream) {
  return launch_dense_mfma<FMT>(a, stream, ws, ws_bytes);
}
template <int FMT>
hipError_t launch_grouped_mma_fmt(const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream) {
  return launch_grouped_mfma<FMT>(a, n_segs, z_ext, stream);
}

template <int FMT>
hipError_t launch_grouped_fmt(const GroupedArgs& a, int n_segs, int z_ext, hipStream_t stream) {
  if (use_mfma_core()) return launch_grouped_mfma<FMT>(a, n_segs, z_ext, stream);
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
    dispatch_bool(a.once != 0, [&](auto ntc) {
      auto kern = grouped_gemv_kernel<FMT, NB, decltype(ntc)::value>;
      err = ensure_lds(kern, lds);
      if (err != hipSuccess) return;
      hipLaunchKernelGGL(kern, grid, dim3(kBlockThreads), lds, stream, a, g, steps);
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}
#endif  // DGPP_GEMV_IMPL

}  // namespace dgpp_amd
