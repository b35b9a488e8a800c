// The routed expert chain of a small decode batch in ONE launch: the gate/up + SwiGLU blocks of every routed
// slot lead a one-dimensional grid, the token-major down + accumulation blocks follow it. Both parts are the
// two-launch kernels' own bodies (slot_gate_up_body, token_down_body): every output bit is the two launches'.
//
// Hand-over inside the launch. A slot's act row is complete when each of its `gu_tiles` gate/up blocks has
// counted itself in on the slot's readiness word; a down wavefront looks at the word of the one slot it reads
// before it fetches the row. No fence is involved (a device-scope fence is an L2 write-back / invalidate on this
// chip): act values leave as agent-scope stores, which are written through to the memory side, a gate/up
// wavefront waits for its stores' acknowledgements before the block's one increment per slot, and the down
// wavefronts read word and row with agent-scope loads, which pass their XCD's L2. Increments carry no return
// value. Every reader increments the word as well, with a wrap at gu_tiles + dn_tiles - 1: the last reader
// of a slot returns its word to zero, so the words are zeroed once by their owner and are at rest between
// launches (a HIP graph replays the launch with no memset node).
//
// Why the wait ends. Workgroups of a one-dimensional grid are handed out in index order, so when the first
// down block is handed out every gate/up block is resident or finished, and resident gate/up blocks wait for
// nothing. Should a runtime ever break that order the wait still ends: it is bounded by `spins` polls, after
// which the wavefront raises `status` and goes on with whatever the row holds (the caller reads `status` at
// its next synchronisation and treats a non-zero value as a failed launch).
//
// Reference: the two launches this stands for are launch_moe_slot_gate_up_swiglu{,_fp4} and launch_moe_slot_down{,_fp4}
// + launch_moe_slot_accum_routed_* (src/kernels/glm_moe_launch.hpp:247-283, :392-407); the reference's own counters
// that return to zero are the stealing pair of its FP4 down kernel (src/kernels/glm_moe.cu:2092-2099).
#pragma once

#include "gemv_kernels.hpp"

namespace dgpp_amd {

// Four wavefronts per SIMD (128 vector registers): the down part keeps two slots' passes in flight per wavefront.
constexpr int kChainWavesPerSimd = 4;

template <int FMT, int NBG, int NBD>
__global__ __launch_bounds__(kBlockThreads, kChainWavesPerSimd) void slot_chain_kernel(ChainArgs c, RowGeom gg, int gu_steps,
                                                                                     RowGeom gd, int dn_steps) {
  extern __shared__ uint4 lds[];
  const int b = static_cast<int>(blockIdx.x);
  const unsigned wrap = static_cast<unsigned>(c.gu_tiles + c.dn.tiles - 1);
  if (b < c.gu_blocks) {
    const int rs = b / c.gu_tiles, tile = b - rs * c.gu_tiles;      // routed slot index t * top_k + j, slot-major
    const int t = rs / c.gu.top_k;
    const SlotPublish pub{c.ready, kReadyStride, wrap};
    slot_gate_up_body<FMT, NBG, kGateUpRun, true, true, kWavesPerBlock, true>(c.gu, gg, gu_steps, lds, rs + t, tile, &pub);
  } else {
    const SlotAwait aw{c.ready, kReadyStride, static_cast<unsigned>(c.gu_tiles), wrap, c.spins, c.status};
    token_down_pair_body<FMT, NBD, true>(c.dn, gd, dn_steps, lds, b - c.gu_blocks, &aw);
  }
}

// The one-token step in ONE launch: every block's first wavefront repeats the router's selection in registers
// (select_gate_up_kernel's way), ids and weights go to LDS behind the stage, and the block goes on as a gate/up or
// a down block of the chain. With one token every block of the grid is resident at once: the down wavefronts'
// first weight passes are in their registers by the time the gate/up blocks have counted themselves in.
// Block 0 stores ids and weights for the caller. n_experts <= 512.
template <int FMT, int NBG, int NBD>
__global__ __launch_bounds__(kBlockThreads, kChainWavesPerSimd) void select_chain_kernel(ChainArgs c, SelectArgs sel, RowGeom gg,
                                                                                         int gu_steps, RowGeom gd, int dn_steps,
                                                                                         int sel_off) {
  extern __shared__ uint4 lds[];
  int32_t* ids = reinterpret_cast<int32_t*>(lds + sel_off);
  float* wts = reinterpret_cast<float*>(ids + kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int K = c.gu.top_k;
  if (threadIdx.x < kWave) {
    int id;
    float w;
    if (sel.n_experts <= 4 * kWave) {
      if (sel.mode == DGPP_ROUTER_SOFTMAX_TOPK)
        rsel::select_token<DGPP_ROUTER_SOFTMAX_TOPK, 4>(sel.scores, sel.biased, sel.n_experts, K, sel.scaling, sel.norm_topk, lane, id, w);
      else
        rsel::select_token<DGPP_ROUTER_SIGMOID_BIAS, 4>(sel.scores, sel.biased, sel.n_experts, K, sel.scaling, sel.norm_topk, lane, id, w);
    } else {
      if (sel.mode == DGPP_ROUTER_SOFTMAX_TOPK)
        rsel::select_token<DGPP_ROUTER_SOFTMAX_TOPK, 8>(sel.scores, sel.biased, sel.n_experts, K, sel.scaling, sel.norm_topk, lane, id, w);
      else
        rsel::select_token<DGPP_ROUTER_SIGMOID_BIAS, 8>(sel.scores, sel.biased, sel.n_experts, K, sel.scaling, sel.norm_topk, lane, id, w);
    }
    if (lane < K) {
      ids[lane] = id;
      wts[lane] = w;
      if (blockIdx.x == 0) {
        sel.ids[lane] = id;
        sel.weights[lane] = w;
      }
    }
  }
  __syncthreads();
  const int b = static_cast<int>(blockIdx.x);
  const unsigned wrap = static_cast<unsigned>(c.gu_tiles + c.dn.tiles - 1);
  if (b < c.gu_blocks) {
    SlotArgs u = c.gu;
    u.ids = ids;
    const int j = b / c.gu_tiles, tile = b - j * c.gu_tiles;
    const SlotPublish pub{c.ready, kReadyStride, wrap};
    slot_gate_up_body<FMT, NBG, 1, true, true, kWavesPerBlock, true>(u, gg, gu_steps, lds, j, tile, &pub);
  } else {
    TokenDownArgs d = c.dn;
    d.ids = ids;
    d.weights = wts;
    const SlotAwait aw{c.ready, kReadyStride, static_cast<unsigned>(c.gu_tiles), wrap, c.spins, c.status};
    token_down_pair_body<FMT, NBD, true>(d, gd, dn_steps, lds, b - c.gu_blocks, &aw);
  }
}

template <int FMT>
hipError_t launch_slot_chain_fmt(const ChainArgs& in, const SelectArgs* sel, hipStream_t stream) {
  ChainArgs c = in;
  const int K = c.gu.top_k, T = c.dn.tokens;
  const RowGeom gg = geom_for<FMT>(c.gu.k), gd = geom_for<FMT>(c.dn.k);
  // gate/up: the two-launch form's block (two row steps for a decode batch, one for one token)
  const int rpw_g = kWave >> gg.l2;
  int gu_steps = 2;
  if (tune_get(kTuneSlotSteps) > 0) gu_steps = tune_get(kTuneSlotSteps);
  const int gu_rows = kWavesPerBlock * rpw_g * gu_steps;
  c.gu_tiles = (c.gu.n + gu_rows - 1) / gu_rows;
  c.gu_blocks = c.gu_tiles * T * K;
  // down: the token-major launch's row tiles
  const int rpw_d = kWave >> gd.l2;
  const long long wave_steps = static_cast<long long>((c.dn.n + rpw_d - 1) / rpw_d) * T * K;
  int dn_steps = static_cast<int>(wave_steps / 16384);
  dn_steps = dn_steps < 2 ? 2 : (dn_steps > 8 ? 8 : dn_steps);
  if (sel != nullptr) dn_steps = 1;   // one token: every down wavefront's only weight pass is issued before it waits
  if (tune_get(kTuneChainDownSteps) > 0) dn_steps = tune_get(kTuneChainDownSteps);
  const int dn_rows = rpw_d * dn_steps;
  c.dn.tiles = (c.dn.n + dn_rows - 1) / dn_rows;
  c.dn.xcd_group = 0;
  {
    const int want = tune_get(kTuneXcdGroup) > 0 ? tune_get(kTuneXcdGroup) : 0;
    if (T > 1 && want > 0 && c.dn.tiles % (8 * want) == 0) c.dn.xcd_group = want;
  }
  c.gu.match = 1;
  c.gu.once = 1;
  c.gu.order = nullptr;
  c.gu.want_shared = 0;
  if (c.spins == 0) c.spins = kChainDefaultSpins;
  const long long blocks = static_cast<long long>(c.gu_blocks) + static_cast<long long>(c.dn.tiles) * T;
  if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  const size_t lds_gu = stage_bytes(kGateUpRun, c.gu.k);
  const size_t lds_dn = static_cast<size_t>(K) * (stage_bytes(1, c.dn.k) + static_cast<size_t>(dn_rows) * sizeof(float));
  const size_t lds_main = ((lds_gu > lds_dn ? lds_gu : lds_dn) + 15) / 16 * 16;
  const size_t lds = lds_main + (sel != nullptr ? 2 * kWave * sizeof(int32_t) : 0);
  hipError_t err = hipSuccess;
  dispatch_nb(gg.nb, [&](auto ng) {
    dispatch_nb(gd.nb, [&](auto nd) {
      constexpr int NBG = decltype(ng)::value, NBD = decltype(nd)::value;
      if constexpr (NBG > 4 || NBD > 4 || NBG == 3 || NBD == 3) {
        err = hipErrorInvalidValue;   // the caller's fit check keeps these pass widths on the two launches
      } else {
        if (sel != nullptr) {
          auto kern = select_chain_kernel<FMT, NBG, NBD>;
          err = ensure_lds(kern, lds);
          if (err == hipSuccess)
            hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(kBlockThreads), lds, stream, c, *sel, gg, gu_steps,
                               gd, dn_steps, static_cast<int>(lds_main / sizeof(uint4)));
        } else {
          auto kern = slot_chain_kernel<FMT, NBG, NBD>;
          err = ensure_lds(kern, lds);
          if (err == hipSuccess)
            hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(kBlockThreads), lds, stream, c, gg, gu_steps, gd,
                               dn_steps);
        }
      }
    });
  });
  return err != hipSuccess ? err : hipGetLastError();
}

}  // namespace dgpp_amd
