// The gated shared expert's decode tail with block-FP8 weights, in two launches:
//   act = swiglu(bf16(x . gate_w), bf16(x . up_w))  and  sw[t] = bf16(sigmoid(bf16(x[t] . g)))     (one launch)
//   out = bf16(fma(sw, act . down_w, routed accumulation))                                         (one launch)
// Every dot is the dense FP8 GEMV's own chain (the same row geometry and row_dots), the SwiGLU is the
// slot kernels' epilogue without clamps, the accumulation is the accumulate kernels' fma, so the tail is
// bitwise the unfused chain of launchers it stands for: two grid GEMVs to BF16, swiglu_clamp, a grid GEMV
// to F32, the shared gate, accumulate, round.
//
// Reference counterparts: src/kernels/qwen_moe.hpp:12-87 (interface), src/kernels/qwen_moe.cu:27-56
// (shared gate), :60-120 (gate/up + SwiGLU), :122-198 (down with the accumulation in the epilogue),
// :343-482 (argument rules). The BF16-weight forms of the same tail are not provided.
#define DGPP_GEMV_IMPL
#include "gemv_kernels.hpp"

#include <string>

#include "../../include/dgpp_amd.h"
#include "capi_errors.hpp"

namespace dgpp_amd {
namespace {

constexpr int kFmt = kFmtFp8F32;
constexpr int kTailMaxTokens = 8;    // src/kernels/qwen_moe.cu:346 (2 * gemv::kMaxRows)
constexpr int kTailMaxTopK = 16;     // src/kernels/qwen_moe.cu:132 (kSharedAccMaxK)

// One half wavefront's shared gate for a token: 32 lanes' strided FP32 partial sums over 16-byte vectors
// (low element of a word, then the high one), the xor tree 16, 8, 4, 2, 1, bf16(logit), bf16(sigmoid):
// the reference's order, src/kernels/qwen_moe.cu:27-56. No gate vector: weight 1.
__device__ __forceinline__ float shared_gate_half(const uint16_t* __restrict__ xrow, const uint16_t* __restrict__ g, int hidden,
                                                  int lane32) {
  if (g == nullptr) return 1.0f;
  const uint4* xv = reinterpret_cast<const uint4*>(xrow);
  const uint4* gv = reinterpret_cast<const uint4*>(g);
  float dot = 0.f;
  for (int v = lane32; v < hidden / 8; v += 32) {
    const uint4 xq = xv[v], gq = gv[v];
    const uint32_t xw[4] = {xq.x, xq.y, xq.z, xq.w};
    const uint32_t gw[4] = {gq.x, gq.y, gq.z, gq.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dot = __builtin_fmaf(bits_f32(xw[i] << 16), bits_f32(gw[i] << 16), dot);
      dot = __builtin_fmaf(bits_f32(xw[i] & 0xffff0000u), bits_f32(gw[i] & 0xffff0000u), dot);
    }
  }
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
  const float logit = bf16_to_f32(f32_to_bf16(dot));
  return bf16_to_f32(f32_to_bf16(sigmoid_f32(logit)));
}

// Tokens 2 * wave and 2 * wave + 1 of a block of four wavefronts: eight tokens a block.
__device__ __forceinline__ void shared_gate_block(const uint16_t* __restrict__ x, size_t x_stride, const uint16_t* __restrict__ g,
                                                  float* __restrict__ w, int first, int tokens, int hidden) {
  const int lane = threadIdx.x & (kWave - 1);
  const int t = first + 2 * static_cast<int>(threadIdx.x >> 6) + (lane >> 5);
  if (t >= tokens) return;
  const float v = shared_gate_half(x + static_cast<size_t>(t) * x_stride, g, hidden, lane & 31);
  if ((lane & 31) == 0) w[t] = v;
}

__global__ __launch_bounds__(kBlockThreads) void shared_gate_kernel(const uint16_t* x, size_t x_stride, const uint16_t* g, float* w,
                                                                    int tokens, int hidden) {
  shared_gate_block(x, x_stride, g, w, static_cast<int>(blockIdx.x) * 2 * kWavesPerBlock, tokens, hidden);
}

struct GateUpArgs {
  const uint16_t* x;
  size_t x_stride;
  MatRef gate, up;
  const uint16_t* g;   // the shared gate's vector, nullable
  uint16_t* act;       // [tokens, n]
  float* sw;           // [tokens]
  int tokens, n, k;    // n = S rows of gate / up, k = H
};

// Blocks [0, gridDim.x - 1): rows of gate and up against the staged token rows. The last block: the gates.
template <int MAXR, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void shared_gate_up_kernel(GateUpArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  if (blockIdx.x == gridDim.x - 1) {
    shared_gate_block(a.x, a.x_stride, a.g, a.sw, 0, a.tokens, a.k);
    return;
  }
  const int chunks = a.k / FmtTraits<kFmt>::kElemsPerChunk;
  stage_activations<kFmt>(a.x, a.x_stride, a.tokens, a.k, lds);
  __syncthreads();
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  int row0 = blockIdx.x * block_rows(g, steps) + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const auto lg = lane_row<kFmt, true>(a.gate, row0, a.n, a.k, g.l2);
    const auto lu = lane_row<kFmt, true>(a.up, row0, a.n, a.k, g.l2);
    float ag[MAXR], au[MAXR];
    row_dots<kFmt, MAXR, NB>(lg, g, a.gate.cs, lds, chunks, a.tokens, ag);
    row_dots<kFmt, MAXR, NB>(lu, g, a.up.cs, lds, chunks, a.tokens, au);
    if (lg.li == 0 && lg.row < a.n) {
#pragma unroll
      for (int r = 0; r < MAXR; ++r)
        if (r < a.tokens) a.act[static_cast<size_t>(r) * a.n + lg.row] = swiglu_bf16(ag[r], au[r], __builtin_inff());
    }
  }
}

struct DownArgs {
  const uint16_t* act;   // [tokens, k]
  MatRef down;           // [n, k]
  const float* sw;       // [tokens]
  const float* acc;      // [tokens, n], or null with the slot form below
  const float* contrib;  // [tokens * (top_k + 1), n]: the per-slot routed down outputs
  const float* weights;  // [tokens, top_k]
  int top_k;
  uint16_t* out;         // [tokens, n]
  int tokens, n, k;      // n = H rows of down, k = S
};

// out[r][h] = bf16(fma(sw[r], act[r] . down[h], a)), a = acc[r][h] or the routed slots' fma chain in slot
// order from zero (src/kernels/qwen_moe.cu:186-196; the order of the accumulate kernel, glm_moe.cu:673-711).
template <int MAXR, int NB>
__global__ __launch_bounds__(kBlockThreads, kMinWavesPerSimd) void shared_down_kernel(DownArgs a, RowGeom g, int steps) {
  extern __shared__ uint4 lds[];
  const int chunks = a.k / FmtTraits<kFmt>::kElemsPerChunk;
  stage_activations<kFmt>(a.act, static_cast<size_t>(a.k), a.tokens, a.k, lds);
  __syncthreads();
  const int rpw = kWave >> g.l2;
  const int wave = threadIdx.x >> 6;
  int row0 = blockIdx.x * block_rows(g, steps) + wave * rpw;
  for (int s = 0; s < steps; ++s, row0 += kWavesPerBlock * rpw) {
    if (row0 >= a.n) break;
    const auto lr = lane_row<kFmt, true>(a.down, row0, a.n, a.k, g.l2);
    float d[MAXR];
    row_dots<kFmt, MAXR, NB>(lr, g, a.down.cs, lds, chunks, a.tokens, d);
    // Every lane of a row's group holds all the dots: lane i of the group finishes token i (and i + group size,
    // ...), so the tokens' accumulation inputs are fetched side by side, each token's slots in one burst.
    if (lr.row < a.n) {
      for (int r = lr.li; r < a.tokens; r += (1 << g.l2)) {
        float mine = d[0];
#pragma unroll
        for (int q = 1; q < MAXR; ++q) mine = q == r ? d[q] : mine;
        float base;
        if (a.contrib != nullptr) {
          float c[kTailMaxTopK], wt[kTailMaxTopK];
#pragma unroll
          for (int j = 0; j < kTailMaxTopK; ++j) {
            const int jj = j < a.top_k ? j : 0;
            c[j] = a.contrib[(static_cast<size_t>(r) * (a.top_k + 1) + jj) * a.n + lr.row];
            wt[j] = a.weights[r * a.top_k + jj];
          }
          base = 0.f;
#pragma unroll
          for (int j = 0; j < kTailMaxTopK; ++j)
            if (j < a.top_k) base = __builtin_fmaf(wt[j], c[j], base);
        } else {
          base = a.acc[static_cast<size_t>(r) * a.n + lr.row];
        }
        a.out[static_cast<size_t>(r) * a.n + lr.row] = f32_to_bf16(__builtin_fmaf(a.sw[r], mine, base));
      }
    }
  }
}

template <class Go>
void dispatch_rows(int tokens, Go&& go) {
  if (tokens == 1) go(std::integral_constant<int, 1>{});
  else if (tokens == 2) go(std::integral_constant<int, 2>{});
  else if (tokens <= 4) go(std::integral_constant<int, 4>{});
  else go(std::integral_constant<int, 8>{});
}

struct Grid {
  RowGeom g;
  int steps;
  unsigned blocks;
};
Grid grid_for(int n, int k) {
  Grid r;
  r.g = geom_for<kFmt>(k);
  const int rows_per_step = kWavesPerBlock * (kWave >> r.g.l2);
  const long long block_steps = (n + rows_per_step - 1) / rows_per_step;
  r.steps = pick_steps(block_steps);
  r.blocks = static_cast<unsigned>((block_steps + r.steps - 1) / r.steps);
  return r;
}

MatRef mat(const uint8_t* payload, const float* scales, int rs, int cs) {
  MatRef m;
  m.payload = payload;
  m.scales = scales;
  m.divisor = 1.f;
  m.rs = rs;
  m.cs = cs;
  return m;
}

hipError_t run_gate_up(const GateUpArgs& a, hipStream_t stream) {
  const Grid gr = grid_for(a.n, a.k);
  const size_t lds = stage_bytes(a.tokens, a.k);
  hipError_t err = hipSuccess;
  dispatch_nb(gr.g.nb, [&](auto nbc) {
    dispatch_rows(a.tokens, [&](auto rc) {
      auto kern = shared_gate_up_kernel<decltype(rc)::value, decltype(nbc)::value>;
      err = ensure_lds(kern, lds);
      if (err == hipSuccess) hipLaunchKernelGGL(kern, dim3(gr.blocks + 1), dim3(kBlockThreads), lds, stream, a, gr.g, gr.steps);
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}

hipError_t run_down(const DownArgs& a, hipStream_t stream) {
  const Grid gr = grid_for(a.n, a.k);
  const size_t lds = stage_bytes(a.tokens, a.k);
  hipError_t err = hipSuccess;
  dispatch_nb(gr.g.nb, [&](auto nbc) {
    dispatch_rows(a.tokens, [&](auto rc) {
      auto kern = shared_down_kernel<decltype(rc)::value, decltype(nbc)::value>;
      err = ensure_lds(kern, lds);
      if (err == hipSuccess) hipLaunchKernelGGL(kern, dim3(gr.blocks), dim3(kBlockThreads), lds, stream, a, gr.g, gr.steps);
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// src/kernels/qwen_moe.cu:377-379.
int check_grid(int rs, int cs, const std::string& who) {
  if (rs < 0 || cs < 4 || cs > 30) return report_invalid(who + ": scale grid (rs >= 0, cs >= 4)");
  return DGPP_OK;
}
// The geometry every entry needs (the reference states it for the one-call tails, src/kernels/qwen_moe.cu:405-413;
// its halves leave it to the caller): at most eight tokens, H and S multiples of 16, 16-byte aligned operands,
// a token row of either width stageable.
int check_shape(int tokens, int H, int S, const std::string& who) {
  if (tokens > kTailMaxTokens) return report_invalid(who + ": tokens beyond the decode rows");
  if (H <= 0 || H % 16 != 0 || S <= 0 || S % 16 != 0 || stage_bytes(tokens, H) > kMaxLdsBytes ||
      stage_bytes(tokens, S) > kMaxLdsBytes)
    return report_invalid(who + ": H and S multiples of 16, 16-byte aligned operands");
  return DGPP_OK;
}

int gate_up(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s, const uint8_t* up_p,
            const float* up_s, const uint16_t* g, uint16_t* act, float* sw, int tokens, int H, int S, void* stream, int rs,
            int cs, const std::string& who) {
  if (!x || !gate_p || !gate_s || !up_p || !up_s || !act || !sw) return report_invalid(who + ": null pointer");
  int rc = check_grid(rs, cs, who);
  if (rc == DGPP_OK) rc = check_shape(tokens, H, S, who);
  if (rc != DGPP_OK) return rc;
  if (x_stride < static_cast<size_t>(H) || (x_stride * 2) % 16 != 0 || !aligned16(x) || !aligned16(g) || !aligned16(gate_p) ||
      !aligned16(up_p) || !aligned16(act))
    return report_invalid(who + ": H and S multiples of 16, 16-byte aligned operands");
  GateUpArgs a;
  a.x = x;
  a.x_stride = x_stride;
  a.gate = mat(gate_p, gate_s, rs, cs);
  a.up = mat(up_p, up_s, rs, cs);
  a.g = g;
  a.act = act;
  a.sw = sw;
  a.tokens = tokens;
  a.n = S;
  a.k = H;
  return report_hip(run_gate_up(a, static_cast<hipStream_t>(stream)), who.c_str());
}

int down(const uint16_t* act, const uint8_t* down_p, const float* down_s, const float* sw, const float* acc,
         const float* contrib, const float* weights, int top_k, bool routed, uint16_t* out, int tokens, int H, int S,
         void* stream, int rs, int cs, const std::string& who) {
  if (!act || !down_p || !down_s || !sw || !out) return report_invalid(who + ": null pointer");
  if (routed) {
    if (!contrib || !weights || top_k <= 0 || top_k > kTailMaxTopK) return report_invalid(who + ": slots");
  } else if (!acc) {
    return report_invalid(who + ": null pointer");
  }
  int rc = check_grid(rs, cs, who);
  if (rc == DGPP_OK) rc = check_shape(tokens, H, S, who);
  if (rc != DGPP_OK) return rc;
  if (!aligned16(act) || !aligned16(down_p)) return report_invalid(who + ": H and S multiples of 16, 16-byte aligned operands");
  DownArgs a;
  a.act = act;
  a.down = mat(down_p, down_s, rs, cs);
  a.sw = sw;
  a.acc = routed ? nullptr : acc;
  a.contrib = routed ? contrib : nullptr;
  a.weights = weights;
  a.top_k = top_k;
  a.out = out;
  a.tokens = tokens;
  a.n = H;
  a.k = S;
  return report_hip(run_down(a, static_cast<hipStream_t>(stream)), who.c_str());
}

}  // namespace
}  // namespace dgpp_amd

using namespace dgpp_amd;

extern "C" {

int dgpp_qwen_moe_shared_gate_bf16(const uint16_t* x, const uint16_t* g, float* w, int tokens, int hidden, void* stream) {
  const std::string who = "qwen_moe_shared_gate";
  if (tokens <= 0) return DGPP_OK;
  if (!x || !w) return report_invalid(who + ": null pointer");
  if (hidden <= 0 || hidden % 8 != 0 || !aligned16(x) || !aligned16(g))
    return report_invalid(who + ": hidden % 8 == 0 and 16-byte aligned x, g required");
  const unsigned blocks = static_cast<unsigned>((tokens + 2 * kWavesPerBlock - 1) / (2 * kWavesPerBlock));
  hipLaunchKernelGGL(shared_gate_kernel, dim3(blocks), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream), x,
                     static_cast<size_t>(hidden), g, w, tokens, hidden);
  return report_hip(hipGetLastError(), who.c_str());
}

int dgpp_qwen_moe_shared_gate_up_decode_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                            const uint8_t* up_p, const float* up_s, const uint16_t* g, uint16_t* act, float* sw,
                                            int tokens, int H, int S, void* stream, int rs, int cs) {
  if (tokens <= 0) return DGPP_OK;
  return gate_up(x, x_stride, gate_p, gate_s, up_p, up_s, g, act, sw, tokens, H, S, stream, rs, cs, "qwen moe shared gate_up fp8");
}
int dgpp_qwen_moe_shared_down_decode_fp8(const uint16_t* act, const uint8_t* down_p, const float* down_s, const float* sw,
                                         const float* acc, uint16_t* out, int tokens, int H, int S, void* stream, int rs,
                                         int cs) {
  if (tokens <= 0) return DGPP_OK;
  return down(act, down_p, down_s, sw, acc, nullptr, nullptr, 0, false, out, tokens, H, S, stream, rs, cs, "qwen moe shared down fp8");
}
int dgpp_qwen_moe_shared_down_decode_routed_fp8(const uint16_t* act, const uint8_t* down_p, const float* down_s, const float* sw,
                                                const float* contrib, const float* weights, int top_k, uint16_t* out,
                                                int tokens, int H, int S, void* stream, int rs, int cs) {
  if (tokens <= 0) return DGPP_OK;
  return down(act, down_p, down_s, sw, nullptr, contrib, weights, top_k, true, out, tokens, H, S, stream, rs, cs,
              "qwen moe shared down routed fp8");
}
int dgpp_qwen_moe_shared_tail_decode_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                         const uint8_t* up_p, const float* up_s, const uint8_t* down_p, const float* down_s,
                                         const uint16_t* g, uint16_t* act, float* sw, const float* acc, uint16_t* out,
                                         int tokens, int H, int S, void* stream, int rs, int cs) {
  const std::string who = "qwen_moe_shared_tail_decode_fp8";
  if (tokens <= 0) return DGPP_OK;
  if (!down_p || !down_s || !acc || !out) return report_invalid(who + ": null pointer");
  const int rc = gate_up(x, x_stride, gate_p, gate_s, up_p, up_s, g, act, sw, tokens, H, S, stream, rs, cs, who);
  if (rc != DGPP_OK) return rc;
  return down(act, down_p, down_s, sw, acc, nullptr, nullptr, 0, false, out, tokens, H, S, stream, rs, cs, who);
}
int dgpp_qwen_moe_shared_tail_decode_routed_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                                const uint8_t* up_p, const float* up_s, const uint8_t* down_p,
                                                const float* down_s, const uint16_t* g, uint16_t* act, float* sw,
                                                const float* contrib, const float* weights, int top_k, uint16_t* out,
                                                int tokens, int H, int S, void* stream, int rs, int cs) {
  const std::string who = "qwen_moe_shared_tail_decode_routed_fp8";
  if (tokens <= 0) return DGPP_OK;
  if (!contrib || !weights || top_k <= 0 || top_k > kTailMaxTopK) return report_invalid(who + ": slots");
  if (!down_p || !down_s || !out) return report_invalid(who + ": null pointer");
  const int rc = gate_up(x, x_stride, gate_p, gate_s, up_p, up_s, g, act, sw, tokens, H, S, stream, rs, cs, who);
  if (rc != DGPP_OK) return rc;
  return down(act, down_p, down_s, sw, nullptr, contrib, weights, top_k, true, out, tokens, H, S, stream, rs, cs, who);
}

}  // extern "C"
