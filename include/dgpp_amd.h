/*
 * dgpp_amd — C ABI of the MI355X (gfx950) quantized MoE expert GEMV path.
 *
 * One `extern "C"` entry point per kernel launcher of the reference's operator surface for this
 * path (src/kernels/glm_moe_launch.hpp, fp4_gemv.hpp, scale_gemm.hpp, fp8_dequant.hpp,
 * minimax.hpp), same argument order and meaning. Differences that the C ABI forces:
 *   - the stream is an opaque `void*` holding a hipStream_t (null = the default stream);
 *   - C++ default arguments are spelled out;
 *   - instead of throwing, every launcher returns DGPP_OK, DGPP_INVALID_ARGUMENT (the
 *     reference's std::invalid_argument: nothing was launched) or DGPP_RUNTIME_ERROR (the
 *     reference's std::runtime_error from a failed runtime call); dgpp_last_error() returns the
 *     message of the calling thread's last failure. include/dgpp_amd.hpp re-throws them.
 *
 * Conventions (reference: src/kernels/glm_moe_launch.hpp:211-243, src/kernels/scale_gemm.hpp:27-36):
 * bf16 travels as uint16_t bit patterns; e4m3 / e2m1 pairs / e8m0 as uint8_t; every pointer is
 * a DEVICE pointer unless the parameter is documented as host; matrices are row-major W[n, k]
 * and the product is D = Act * W^T; strides are in ELEMENTS; launchers are asynchronous on the
 * given stream, allocate nothing, never synchronise, and are deterministic run to run.
 */
#ifndef DGPP_AMD_H
#define DGPP_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DGPP_OK 0
#define DGPP_INVALID_ARGUMENT 1
#define DGPP_RUNTIME_ERROR 2

/* Message of the calling thread's most recent failed call ("" when none). */
const char* dgpp_last_error(void);
/* "gfx950" — the only architecture the library carries code for. */
const char* dgpp_target_arch(void);

/* ---- POD types shared with device code -------------------------------------------------- */

/* Device-side expert table entry, read by the slot and grouped kernels.
 * Layout-identical (96 bytes, same offsets) to the reference's MoeExpertView,
 * src/models/glm/moe.hpp:232-292. Fields the path does not use are kept as reserved space. */
typedef struct DgppMoeExpertView {
  const uint8_t* payload;     /*  0  fp8: e4m3 [n, k]; fp4: e2m1 pairs [n, k/2]            */
  const float* scales;        /*  8  fp8: F32 block scales (fp4: null)                     */
  const uint8_t* fp4_scales;  /* 16  NVFP4: e4m3 [n, k/16]; MXFP4: e8m0 [n, k/32]          */
  const float* fp4_global;    /* 24  NVFP4: the matrix's F32 global scale (MXFP4: null)    */
  int32_t scale_shift_rows;   /* 32  fp8 scale grid, log2 block rows (7 = 128)             */
  int32_t scale_shift_cols;   /* 36  fp8 scale grid, log2 block cols                       */
  int32_t fp4_group;          /* 40  16 = NVFP4, 32 = MXFP4                                */
  int32_t reserved0;          /* 44                                                        */
  const void* reserved1;      /* 48  (reference: packed_scales)                            */
  int32_t reserved2[2];       /* 56  (reference: bits, packed_scale_fmt)                   */
  const void* reserved3[2];   /* 64  (reference: exl3_suh, exl3_svh)                       */
  int32_t reserved4[4];       /* 80  (reference: exl3_bits, exl3_rows, exl3_cols, pad)     */
} DgppMoeExpertView;

/* src/kernels/glm_moe_launch.hpp:67-71 */
typedef struct DgppMoeSegment {
  int32_t row0;   /* first row of the segment in act / out */
  int32_t rows;   /* rows in the segment */
  int32_t expert; /* view-table expert index (the shared expert last) */
} DgppMoeSegment;

/* src/kernels/glm_moe_launch.hpp:151-154 */
typedef struct DgppMoeTile {
  int32_t seg; /* index into the segment table */
  int32_t m0;  /* first row of the tile within the segment */
} DgppMoeTile;

/* src/models/quant_matrix.hpp:117-138 (GlmFp4Matrix), same 56-byte layout. */
typedef struct DgppFp4Matrix {
  const uint8_t* payload;     /* U8 [rows, cols/2], low nibble = even element */
  const uint8_t* scales;      /* e4m3 [rows, cols/16] or e8m0 [rows, cols/32] */
  const float* global_scale;  /* F32 [1] on the device; null under MXFP4 */
  int64_t rows;
  int64_t cols;               /* logical K (elements) */
  int32_t scale_group;        /* 16: NVFP4, 32: MXFP4 */
  int32_t reserved0;
  const void* reserved1;      /* (reference: tma) */
} DgppFp4Matrix;

/* Router scoring rule, src/models/glm/moe.hpp:49. */
#define DGPP_ROUTER_SIGMOID_BIAS 0
#define DGPP_ROUTER_SOFTMAX_TOPK 1
#define DGPP_ROUTER_SQRT_SOFTPLUS_BIAS 2

/* The router-relevant fields of the reference's GlmMoeConfig, src/models/glm/moe.hpp:51-134.
 * dgpp_moe_config_validate applies validate_config's rules (moe.hpp:119-133). */
typedef struct DgppMoeConfig {
  int32_t hidden;
  int32_t inter;
  int32_t n_experts;
  int32_t top_k;
  int32_t n_shared_experts;
  float routed_scaling_factor;
  int32_t norm_topk_prob;
  float swiglu_limit;
  int32_t router_mode;
} DgppMoeConfig;
int dgpp_moe_config_validate(const DgppMoeConfig* cfg);

/* ---- router ------------------------------------------------------------------------------ */
/* src/kernels/glm_moe_launch.hpp:23 (launch_moe_router). counters (nullable) is accepted for signature parity; the
 * two-launch form (score rows, then the selection) runs either way and the counters stay zero - hosts that want the
 * selection off the critical path run it inside a later launch (the extensions below). allow_tiled != 0: from 32 rows
 * on (the reference: 16) the score rows come from the token-tiled kernel (a gate row fetched once per two or four
 * tokens), bit for bit the one-row form's values (src/kernels/glm_moe.cu:735-760, :848-866). */
int dgpp_launch_moe_router(const uint16_t* hidden, const uint16_t* gate, const float* bias,
                           int32_t* ids, float* weights, float* scores, float* biased,
                           const DgppMoeConfig* cfg, int tokens, void* stream, int* counters,
                           int allow_tiled);
/* src/kernels/glm_moe_launch.hpp:30-39 (launch_moe_hash_routes): after the router has left every expert's score in
 * `scores`, the routes are replaced - ids [n_tokens, top_k] = row tokens[t] of tid2eid (int32 [vocab, top_k], rows
 * ascending), weights the scores at those ids normalised and scaled as the selection does. tokens: device int64
 * [n_tokens]; a token id outside [0, vocab) reads row 0. Refused in softmax mode (the router leaves logits there). */
int dgpp_launch_moe_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int32_t* ids,
                                float* weights, const DgppMoeConfig* cfg, int vocab, int n_tokens, void* stream);
/* Extension (no counterpart in the reference): step 1 of dgpp_launch_moe_router alone - the score rows (`scores`,
 * and `biased` = scores + bias, or the same values in softmax mode) without the selection, for hosts that run the
 * selection inside a later launch (dgpp_launch_moe_router_select_order, dgpp_launch_moe_select_gate_up_swiglu). */
int dgpp_launch_moe_router_dots(const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                                float* biased, const DgppMoeConfig* cfg, int tokens, void* stream);

/* The selection half of launch_moe_router alone (src/kernels/glm_moe.cu:314-329,
 * moe_router_select_kernel): scores / biased f32 [tokens, n_experts] already on the device
 * (softmax mode: the bf16-rounded logits in both) -> ids ascending, weights. */
int dgpp_launch_moe_router_select(const float* scores, const float* biased, int32_t* ids,
                                  float* weights, const DgppMoeConfig* cfg, int tokens,
                                  void* stream);

/* ---- elementwise pieces -------------------------------------------------------------------- */
/* Extension: the selection of dgpp_launch_moe_router_select and, when `order` is given, the slot
 * order of dgpp_launch_moe_slot_order (same outputs, bit for bit) in one launch for decode batches
 * (tokens <= 16 and n_experts <= 512; larger problems run the two kernels). */
int dgpp_launch_moe_router_select_order(const float* scores, const float* biased, int32_t* ids, float* weights,
                                        int32_t* order, const DgppMoeConfig* cfg, int tokens, int shared_early,
                                        void* stream);

/* src/kernels/glm_moe_launch.hpp:43 */
int dgpp_launch_moe_swiglu_clamp(const uint16_t* gate, const uint16_t* up, uint16_t* out,
                                 int64_t n, float limit, void* stream);
/* src/kernels/glm_moe_launch.hpp:48 */
int dgpp_launch_moe_gather_rows(const uint16_t* src, const int32_t* rows, uint16_t* dst,
                                int n_rows, int hidden, void* stream);
/* src/kernels/glm_moe_launch.hpp:56 */
int dgpp_launch_moe_accum(float* acc, const float* y, const int32_t* rows,
                          const float* row_weights, int n_rows, int hidden, void* stream);
/* src/kernels/glm_moe_launch.hpp:195 */
int dgpp_launch_moe_round_bf16(uint16_t* out, const float* acc, int64_t n, void* stream);

/* ---- grouping ------------------------------------------------------------------------------- */
/* src/kernels/glm_moe_launch.hpp:134 */
int dgpp_launch_moe_segment(const int32_t* ids, int tokens, int top_k, int n_experts,
                            int32_t* rows, int32_t* slot_row, DgppMoeSegment* segs, void* stream);
/* src/kernels/glm_moe_launch.hpp:155-160 */
int dgpp_moe_tile_list_capacity(int n_segs, int total_rows, int tile_rows);
int dgpp_launch_moe_tile_list(const DgppMoeSegment* segs, int n_segs, int tile_rows,
                              DgppMoeTile* tiles, int32_t* count, void* stream);
/* src/kernels/glm_moe_launch.hpp:244; runs (nullable) holds slots + dgpp_moe_run_groups_max(slots)
 * entries (glm_moe_launch.hpp:207-209). */
int dgpp_moe_run_groups_max(int slots);
int dgpp_launch_moe_slot_order(const int32_t* ids, int32_t* order, int slots, int top_k,
                               int n_experts, void* stream, int shared_early, int32_t* runs);
/* src/kernels/minimax.hpp:56-60 (minimax_router; kernels src/kernels/minimax.cu:397-440): the MiniMax router. x: BF16
 * token rows [rows, hidden]; gate: FP32 [experts, hidden]; scores (out) [rows, experts] = sigmoid of the FP32 dot. The
 * top-k is taken by scores + bias (strict '>' : the lower id wins a tie), ids come back ascending, and
 * weights = score / max(sum of the picked scores in id order, 1e-20) * factor, FP32, never narrowed. rows <= 0 returns
 * at once; experts <= 0, topk outside 1..16 or above experts is an invalid argument. At most 4096 experts. */
int dgpp_minimax_router(const uint16_t* x, const float* gate, const float* bias, int rows, int hidden, int experts, int topk,
                        float factor, float* scores, int32_t* ids, float* weights, void* stream);

/* src/kernels/minimax.hpp:11 */
int dgpp_minimax_compact_segments(const DgppMoeSegment* input, DgppMoeSegment* output,
                                  int experts, int capacity, void* stream);

/* ---- ordered accumulation -------------------------------------------------------------------- */
/* src/kernels/glm_moe_launch.hpp:168-180 */
int dgpp_launch_moe_accum_ordered(uint16_t* out, const float* down, size_t down_stride,
                                  const int32_t* slot_row, const int32_t* slot_ids,
                                  const float* slot_w, int shared_row0, int tokens, int top_k,
                                  int hidden, void* stream);
int dgpp_launch_moe_accum_ordered_f32(float* out, const float* down, size_t down_stride,
                                      const int32_t* slot_row, const int32_t* slot_ids,
                                      const float* slot_w, int shared_row0, int tokens, int top_k,
                                      int hidden, void* stream);
/* src/kernels/glm_moe_launch.hpp:182-191: the same chain over BF16 down rows (the W4A4 grouped chain; no shared row),
 * rounded to BF16 or left in FP32. down_stride in BF16 elements. */
int dgpp_launch_moe_accum_ordered_bf16down(uint16_t* out, const uint16_t* down, size_t down_stride, const int32_t* slot_row,
                                           const int32_t* slot_ids, const float* slot_w, int tokens, int top_k, int hidden,
                                           void* stream);
int dgpp_launch_moe_accum_ordered_f32_bf16down(float* out, const uint16_t* down, size_t down_stride, const int32_t* slot_row,
                                               const int32_t* slot_ids, const float* slot_w, int tokens, int top_k, int hidden,
                                               void* stream);
/* src/kernels/glm_moe_launch.hpp:273-283 */
int dgpp_launch_moe_slot_accum(uint16_t* out, const float* contrib, const float* weights,
                               int tokens, int hidden, int top_k, void* stream);
int dgpp_launch_moe_slot_accum_routed_f32(float* out, const float* contrib, const float* weights,
                                          int tokens, int hidden, int top_k, void* stream);

/* No counterpart in the reference: launch_moe_slot_accum_routed_f32 followed by launch_moe_round_bf16
 * (src/kernels/glm_moe_launch.hpp:280, :195) in ONE launch — the routed chain alone rounded once to
 * bf16, bit for bit the two-launch form. */
int dgpp_launch_moe_slot_accum_routed_bf16(uint16_t* out, const float* contrib, const float* weights,
                                           int tokens, int hidden, int top_k, void* stream);

/* ---- FP8 block-scaled decode-slot kernels ------------------------------------------------------ */
/* src/kernels/glm_moe_launch.hpp:247-253 */
int dgpp_launch_moe_slot_gate_up_swiglu(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                        const int32_t* order, const DgppMoeExpertView* views,
                                        int n_routed, int k_routed, int n_shared, int k_shared,
                                        const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                        const uint8_t* sh_up_payload, const float* sh_up_scales,
                                        uint16_t* act, int act_stride, int slots, int top_k,
                                        float limit, void* stream, int sh_rs, int sh_cs);
/* src/kernels/glm_moe_launch.hpp:258-265 */
int dgpp_launch_moe_slot_down(const uint16_t* act, size_t act_stride, const int32_t* ids,
                              const int32_t* order, const DgppMoeExpertView* views, int n_routed,
                              int k_routed, int n_shared, int k_shared, const uint8_t* sh_payload,
                              const float* sh_scales, float* out, int out_stride, int slots,
                              int top_k, void* stream, int sh_rs, int sh_cs);

/* Extensions (no counterpart in the reference): the four decode-slot launchers above and below (gate/up and down,
 * FP8 and FP4) run a routed pass and, with n_shared > 0, a shared pass: two launches that touch disjoint slot rows.
 * The *_ex forms take the reference launcher's arguments unchanged and then
 *   passes       1 the routed pass, 2 the shared pass, 3 both (what the plain launcher runs), so that a host can put
 *                the shared expert's passes on a second stream beside the routed ones; same checks, same bits per pass;
 *   acc_weights, acc_out (down launchers only, both or neither): the shared pass ends with the token's accumulation
 *                instead of a dgpp_launch_moe_slot_accum launch. `out` must hold the routed slots' finished rows by the
 *                time the shared pass runs (the same call's routed pass, or an earlier one on the stream); the shared
 *                pass then stores no slot row but the token's row - a = 0; a = fma(acc_weights[t, j], out[slot j], a)
 *                for j ascending; a = fma(1, shared dot, a); one rounding - to acc_out [tokens, n_shared] (bf16).
 *                Same bits as the two launches.
 * A request that cannot be honoured is DGPP_INVALID_ARGUMENT and nothing is launched: passes outside 1..3, the shared
 * pass alone without a shared expert, an accumulation without the shared pass that would write it. */
int dgpp_launch_moe_slot_gate_up_swiglu_ex(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                           const int32_t* order, const DgppMoeExpertView* views,
                                           int n_routed, int k_routed, int n_shared, int k_shared,
                                           const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                           const uint8_t* sh_up_payload, const float* sh_up_scales,
                                           uint16_t* act, int act_stride, int slots, int top_k,
                                           float limit, void* stream, int sh_rs, int sh_cs, int passes);
int dgpp_launch_moe_slot_down_ex(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                 const int32_t* order, const DgppMoeExpertView* views, int n_routed,
                                 int k_routed, int n_shared, int k_shared, const uint8_t* sh_payload,
                                 const float* sh_scales, float* out, int out_stride, int slots,
                                 int top_k, void* stream, int sh_rs, int sh_cs, int passes,
                                 const float* acc_weights, uint16_t* acc_out);
int dgpp_launch_moe_slot_gate_up_swiglu_fp4_ex(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                               const int32_t* order, const DgppMoeExpertView* views,
                                               int n_routed, int k_routed, int n_shared, int k_shared,
                                               const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                               const uint8_t* sh_up_payload, const float* sh_up_scales,
                                               uint16_t* act, int act_stride, int slots, int top_k,
                                               float limit, void* stream, int shared_view_base,
                                               int fp4_group, int sh_rs, int sh_cs, int passes);
int dgpp_launch_moe_slot_down_fp4_ex(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                     const int32_t* order, const DgppMoeExpertView* views, int n_routed,
                                     int k_routed, int n_shared, int k_shared, const uint8_t* sh_payload,
                                     const float* sh_scales, float* out, int out_stride, int slots,
                                     int top_k, void* stream, int shared_view_base, int fp4_group,
                                     int sh_rs, int sh_cs, int* tile_counter, int passes,
                                     const float* acc_weights, uint16_t* acc_out);

/* Extension (no counterpart in the reference): dgpp_launch_moe_router_select followed by the routed pass of
 * dgpp_launch_moe_slot_gate_up_swiglu / _fp4 (order == NULL, no shared expert; slots = tokens * (top_k + 1)),
 * same outputs bit for bit. For ONE token (n_experts <= 512, k <= 4096, 16-byte-aligned row) this is one launch:
 * the first wavefront of every gate/up block repeats the selection in registers, block (0, 0) stores `ids` and
 * `weights` for the launches that follow. Any other call runs the two launchers. */
int dgpp_launch_moe_select_gate_up_swiglu(const float* scores, const float* biased, int32_t* ids, float* weights,
                                          const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                          const DgppMoeExpertView* views, int n_routed, int k_routed,
                                          uint16_t* act, int act_stride, float limit, void* stream);
int dgpp_launch_moe_select_gate_up_swiglu_fp4(const float* scores, const float* biased, int32_t* ids,
                                              float* weights, const DgppMoeConfig* cfg, int tokens,
                                              const uint16_t* x, size_t x_stride, const DgppMoeExpertView* views,
                                              int n_routed, int k_routed, uint16_t* act, int act_stride,
                                              float limit, void* stream, int fp4_group);

/* ---- NVFP4 / MXFP4 decode-slot kernels ----------------------------------------------------------- */
/* src/kernels/glm_moe_launch.hpp:392-399 */
int dgpp_launch_moe_slot_gate_up_swiglu_fp4(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                            const int32_t* order, const DgppMoeExpertView* views,
                                            int n_routed, int k_routed, int n_shared, int k_shared,
                                            const uint8_t* sh_gate_payload,
                                            const float* sh_gate_scales,
                                            const uint8_t* sh_up_payload, const float* sh_up_scales,
                                            uint16_t* act, int act_stride, int slots, int top_k,
                                            float limit, void* stream, int shared_view_base,
                                            int fp4_group, int sh_rs, int sh_cs);
/* src/kernels/glm_moe_launch.hpp:409-425 (launch_moe_slot_gate_up_swiglu_mixed): the per-projection form's gate/up
 * launch - one projection of every routed expert block-FP8 (its entry's payload / scales / scale shifts), the other
 * NVFP4 (payload / fp4_scales / fp4_global), gate_fp4 != 0 naming the gate as the NVFP4 one. Each dot is bitwise its
 * uniform launcher's; the SwiGLU has the same rounding points. fp4_group must be 16; k in the FP4 core's accepted
 * set and a multiple of 16. The shared slots (n_shared > 0: an FP8 expert on the launch arguments) run as the FP4
 * launcher's do. */
int dgpp_launch_moe_slot_gate_up_swiglu_mixed(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                              const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                              int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                              const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                              int act_stride, int slots, int top_k, float limit, int gate_fp4, int fp4_group,
                                              void* stream, int sh_rs, int sh_cs);
/* src/kernels/glm_moe_launch.hpp:400-408. tile_counter (two device ints zeroed once by the
 * caller) is accepted for signature parity and left untouched: this build's down kernel uses a
 * static grid. */
int dgpp_launch_moe_slot_down_fp4(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                  const int32_t* order, const DgppMoeExpertView* views,
                                  int n_routed, int k_routed, int n_shared, int k_shared,
                                  const uint8_t* sh_payload, const float* sh_scales, float* out,
                                  int out_stride, int slots, int top_k, void* stream,
                                  int shared_view_base, int fp4_group, int sh_rs, int sh_cs,
                                  int* tile_counter);

/* ---- grouped (segment-major) GEMV twins ------------------------------------------------------------ */
/* Extension (no counterpart in the reference, which runs launch_moe_slot_down* and
 * launch_moe_slot_accum_routed_* back to back): the routed slots' down projection AND the token's ordered
 * accumulation chain in one launch, token-major (one wavefront per routed slot of a token, the top_k partial
 * rows meet in LDS). act: the slot activation rows of launch_moe_slot_gate_up_swiglu* (slot = t * (top_k + 1)
 * + j); out_f32 (when given) or out_bf16: [tokens, n]. Bit-identical to the two-launch form. Routed slots
 * only: a shared expert is chained separately. */
int dgpp_launch_moe_slot_down_accum(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                    const DgppMoeExpertView* views, int n, int k, int tokens, int top_k,
                                    const float* weights, uint16_t* out_bf16, float* out_f32, void* stream);
int dgpp_launch_moe_slot_down_accum_fp4(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                        const DgppMoeExpertView* views, int n, int k, int tokens, int top_k,
                                        const float* weights, uint16_t* out_bf16, float* out_f32, void* stream,
                                        int fp4_group);

/* Extension (no counterpart in the reference, whose decode walk runs launch_moe_slot_gate_up_swiglu*,
 * launch_moe_slot_down* and launch_moe_slot_accum_routed_* back to back, src/models/glm/moe_layer.cpp:1641-1677):
 * the routed experts' whole chain of a small decode batch in ONE launch. The gate/up + SwiGLU blocks lead the
 * grid, the token-major down + accumulation blocks follow it and read a slot's act row once the slot's
 * readiness word says that every gate/up block that serves it has stored its values. Bit-identical to the
 * launches it stands for. x: token rows [tokens, x_stride]; act: scratch [tokens * (top_k + 1), act_stride]
 * (slot = t * (top_k + 1) + j, as the slot launchers lay it out); weights: [tokens, top_k]; out_f32 (when given)
 * or out_bf16: [tokens, hidden]. `ready`: dgpp_moe_slot_chain_ready_bytes(tokens, top_k) bytes of device memory the
 * caller zeroes ONCE; every launch leaves them zero (as the reference's counters are left,
 * src/kernels/glm_moe.cu:2092-2099), so a captured launch replays without a memset. `status`: one device int the
 * caller zeroes once; a wavefront whose bounded wait (`spins` polls, 0 = the default) ran out raises it and
 * finishes with whatever the row held — a non-zero status after a synchronisation means the launch's output
 * is invalid (and `ready` must be zeroed again). Launches that share `ready` must not overlap. Problems outside
 * the one-launch form (more than 128 routed slots, top_k above 8, rows that do not fit the register stages,
 * ready or status null) run as the launches above, same bits. Routed slots only. */
size_t dgpp_moe_slot_chain_ready_bytes(int tokens, int top_k);
int dgpp_launch_moe_slot_chain(const uint16_t* x, size_t x_stride, const int32_t* ids, const DgppMoeExpertView* views,
                               int inter, int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                               const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                               unsigned spins, void* stream);
int dgpp_launch_moe_slot_chain_fp4(const uint16_t* x, size_t x_stride, const int32_t* ids, const DgppMoeExpertView* views,
                                   int inter, int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                                   const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                   unsigned spins, void* stream, int fp4_group);

/* The same with the router's selection inside the launch (the reference's fused form selects inside its router
 * launch, src/kernels/glm_moe.cu:840-890; here a one-token step is ONE launch from score rows to the output row):
 * every block's first wavefront repeats the selection, block 0 stores ids / weights [tokens, top_k] for the caller.
 * One token and at most 512 experts take that form; anything else runs dgpp_launch_moe_select_gate_up_swiglu* (or the
 * selection alone) and goes on as dgpp_launch_moe_slot_chain* would. Same bits. */
int dgpp_launch_moe_select_slot_chain(const float* scores, const float* biased, int32_t* ids, float* weights,
                                      const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                      const DgppMoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride,
                                      float limit, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                      unsigned spins, void* stream);
int dgpp_launch_moe_select_slot_chain_fp4(const float* scores, const float* biased, int32_t* ids, float* weights,
                                          const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                          const DgppMoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride,
                                          float limit, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                          unsigned spins, void* stream, int fp4_group);

/* src/kernels/glm_moe_launch.hpp:77-87 */
int dgpp_launch_moe_grouped_gemv_bf16(const uint16_t* act, size_t act_stride,
                                      const DgppMoeSegment* segs, int n_segs, int max_rows,
                                      int rows_per_block, const DgppMoeExpertView* views, int which,
                                      uint16_t* out, size_t out_stride, int n, int k, void* stream);
int dgpp_launch_moe_grouped_gemv_f32(const uint16_t* act, size_t act_stride,
                                     const DgppMoeSegment* segs, int n_segs, int max_rows,
                                     int rows_per_block, const DgppMoeExpertView* views, int which,
                                     float* out, size_t out_stride, int n, int k, void* stream);
/* src/kernels/glm_moe_launch.hpp:375-386 */
int dgpp_launch_moe_grouped_gemv_fp4_bf16(const uint16_t* act, size_t act_stride,
                                          const DgppMoeSegment* segs, int n_segs, int max_rows,
                                          int rows_per_block, const DgppMoeExpertView* views,
                                          int which, uint16_t* out, size_t out_stride, int n, int k,
                                          void* stream, int fp4_group);
int dgpp_launch_moe_grouped_gemv_fp4_f32(const uint16_t* act, size_t act_stride,
                                         const DgppMoeSegment* segs, int n_segs, int max_rows,
                                         int rows_per_block, const DgppMoeExpertView* views,
                                         int which, float* out, size_t out_stride, int n, int k,
                                         void* stream, int fp4_group);

/* ---- dense NVFP4 / MXFP4 projection GEMV -------------------------------------------------------------- */
/* ---- matrix-core launchers ------------------------------------------------------------------
 * The reference's tensor-core forms of the same products (src/kernels/glm_moe_launch.hpp:103-125 dense and
 * grouped FP8, :311-345 grouped and dense FP4; src/kernels/mma_gemv.hpp:65-85 FP8 with a scale grid given
 * as shifts, F32 or E8M0). Here they run on v_mfma_f32_16x16x32_bf16: 16 activation rows ride on one pass
 * over the weights, any m (16-row tiles). A (weight row, activation row) result does not depend on m, on
 * the launcher (dense == grouped == split form, bit for bit) or on `ws`; it is NOT bitwise the GEMV
 * launchers' (another summation order) and is held to the same oracle tolerance.
 * act_rows (nullable): segment row i reads activation row act_rows[i] (the gather folded in).
 * ws / ws_bytes (nullable): room for parts(k) * m * n floats lets an under-filled grid run the K parts in
 * separate blocks plus one folding launch. rows_per_block: segment rows per z block (0 = all).
 * tile_rows is accepted for the signature and ignored. */
int dgpp_launch_dense_mma_bf16(const uint16_t* act, size_t act_stride, const uint8_t* payload, const float* scales,
                               uint16_t* out, int m, int n, int k, void* stream, size_t out_stride);
int dgpp_launch_dense_mma_f32(const uint16_t* act, size_t act_stride, const uint8_t* payload, const float* scales,
                              float* out, int m, int n, int k, void* stream, size_t out_stride);
int dgpp_launch_dense_mma_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, uint16_t* out, int m,
                                   int n, int k, void* stream);
int dgpp_launch_dense_mma_fp4_f32(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, float* out, int m, int n,
                                  int k, void* stream);
/* Extension: the FP4 dense form with the scale-grid launchers' output stride and workspace arguments. */
int dgpp_launch_mma_gemv_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, uint16_t* out, int m,
                                  int n, int k, size_t out_stride, void* stream, void* ws, size_t ws_bytes);
int dgpp_launch_mma_gemv_fp4_f32(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, float* out, int m, int n,
                                 int k, size_t out_stride, void* stream, void* ws, size_t ws_bytes);
/* No counterpart in the reference. dgpp_launch_mma_gemv_fp4_bf16 for callers that cannot allocate a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid allocation): the split-K partial sums go to a
 * workspace of DGPP_STATIC_SCRATCH_BYTES that the library holds in a file-scope device array (each GPU the library runs
 * on keeps its own copy until the process ends). The call allocates nothing and gives dgpp_launch_mma_gemv_fp4_bf16's
 * bits. Only launches that would run split use the workspace (more than one K part: parts = 4 from k = 4096, 2 from
 * k = 2048; and fewer than 1024 tiles of 64 weight rows x 16 activation rows); of those, parts(k) * m * n floats
 * beyond the static workspace are refused with DGPP_INVALID_ARGUMENT. Every other launch runs unsplit, uses no
 * workspace and is never refused for its size. Every split call on a GPU shares that GPU's array, so the array is
 * BOUND to the stream of the first split call: a split call on another stream of that GPU is refused with
 * DGPP_INVALID_ARGUMENT (calls on two streams could overlap and race on the array; calls on one stream follow each
 * other) until dgpp_static_scratch_release() - to be called once the bound stream's work is done - frees the
 * binding. The first split call on a device looks the array's address up. */
#define DGPP_STATIC_SCRATCH_BYTES (8u << 20)
int dgpp_launch_mma_gemv_fp4_bf16_static(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, uint16_t* out,
                                         int m, int n, int k, size_t out_stride, void* stream);
int dgpp_static_scratch_release(void);
/* src/kernels/mma_gemv.hpp:70-94 (launch_mma_gemv_fp8{,e8m0}_{bf16,f32}): the reference's streaming tensor-core GEMV for
 * FP8 weights. The same dispatch as dgpp_launch_scale_gemm_bf16 here: small batches run on the vector core where that
 * is the faster form on this chip (always up to four rows; five to eight rows without a workspace unless the matrix is
 * large), the rest on the matrix core with `ws` as its split-K workspace. The two cores differ in fp32 summation order;
 * both meet the same tolerance against the fp64 oracle. */
int dgpp_launch_mma_gemv_fp8_bf16(const uint16_t* act, size_t act_stride, const uint8_t* w, const float* scales,
                                  uint16_t* out, int m, int n, int k, size_t out_stride, int rs, int cs, void* stream,
                                  void* ws, size_t ws_bytes);
int dgpp_launch_mma_gemv_fp8_f32(const uint16_t* act, size_t act_stride, const uint8_t* w, const float* scales, float* out,
                                 int m, int n, int k, size_t out_stride, int rs, int cs, void* stream, void* ws,
                                 size_t ws_bytes);
int dgpp_launch_mma_gemv_fp8e8m0_bf16(const uint16_t* act, size_t act_stride, const uint8_t* w, const uint8_t* scales,
                                      uint16_t* out, int m, int n, int k, size_t out_stride, int rs, int cs, void* stream,
                                      void* ws, size_t ws_bytes);
int dgpp_launch_mma_gemv_fp8e8m0_f32(const uint16_t* act, size_t act_stride, const uint8_t* w, const uint8_t* scales,
                                     float* out, int m, int n, int k, size_t out_stride, int rs, int cs, void* stream,
                                     void* ws, size_t ws_bytes);
int dgpp_launch_moe_grouped_mma_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                     int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                     uint16_t* out, size_t out_stride, int n, int k, void* stream,
                                     const int32_t* act_rows);
int dgpp_launch_moe_grouped_mma_f32(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                    int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which, float* out,
                                    size_t out_stride, int n, int k, void* stream, const int32_t* act_rows);
/* src/kernels/mma_gemv.hpp:103-104, :119-130 (mma_gemv_shape_ok, mma_gemv_pair_ok, launch_mma_gemv_fp8_bf16_pair): two
 * FP8 projections of one k against one batch in ONE launch - two dependent-free GEMVs sharing one ramp and drain.
 * Each row's bits are those of dgpp_launch_mma_gemv_fp8_bf16 on its own problem (up to eight rows: both problems in one
 * vector-core launch; more: one matrix-core launch). act_stride is both activations';
 * ws (nullable here) holds both problems' K-part sums: parts(k) * m * (n0 + n1) floats. pair_ok mirrors the reference's
 * conditions that carry over (a workspace, 1 <= m <= 32, both shapes taken, the workspace large enough). */
int dgpp_mma_gemv_shape_ok(const void* w, const void* act, size_t act_stride, int m, int k);
int dgpp_mma_gemv_pair_ok(const void* w0, const void* w1, const uint16_t* a0, const uint16_t* a1, size_t act_stride, int m,
                          int n0, int n1, int k, void* ws, size_t ws_bytes);
int dgpp_launch_mma_gemv_fp8_bf16_pair(const uint16_t* a0, const uint8_t* w0, const float* s0, uint16_t* o0, int n0,
                                       size_t stride0, const uint16_t* a1, const uint8_t* w1, const float* s1, uint16_t* o1,
                                       int n1, size_t stride1, size_t act_stride, int m, int k, int rs, int cs, void* stream,
                                       void* ws, size_t ws_bytes);
/* src/kernels/mma_gemv.hpp:86-95 (launch_mma_gemv_fp8_swiglu_f32): out = swiglu(gate, up) x W^T with the activation
 * computed as the rows are staged; bitwise dgpp_launch_moe_swiglu_clamp followed by dgpp_launch_mma_gemv_fp8_f32
 * (unsplit). gate / up: bf16 [m, act_stride], 16-byte aligned rows. */
int dgpp_launch_mma_gemv_fp8_swiglu_f32(const uint16_t* gate, const uint16_t* up, float limit, size_t act_stride,
                                        const uint8_t* w, const float* scales, float* out, int m, int n, int k,
                                        size_t out_stride, int rs, int cs, void* stream);
/* src/kernels/glm_moe_launch.hpp:354-357 (launch_dense_mma_fp4_prod_bf16): the rows of ONE device-resident segment
 * against views[seg->expert * 3 + which]; out [m, n]. The grouped matrix-core kernel's chain. */
int dgpp_launch_dense_mma_fp4_prod_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* seg,
                                        const DgppMoeExpertView* views, int which, uint16_t* out, int m, int n, int k,
                                        void* stream, int fp4_group);
/* src/kernels/glm_moe_launch.hpp:359-365, dense_fp4_decode.cu:297-308: the small dense NVFP4 shard form. The shape
 * predicate is the reference's (fp4_group 16, 1 <= m <= 16, n and k <= 17408, k % 128 == 0); a shape inside it runs as
 * dgpp_launch_dense_mma_fp4_prod_bf16 does (the reference's decode form keeps the production kernel's chain) and sets
 * *launched to 1; outside it nothing runs and *launched is 0, as the reference returns false. */
int dgpp_dense_fp4_decode_shape(int m, int n, int k, int fp4_group);
int dgpp_try_dense_fp4_decode_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* seg,
                                   const DgppMoeExpertView* views, int which, uint16_t* out, int m, int n, int k,
                                   void* stream, int fp4_group, int* launched);
/* src/kernels/glm_moe_launch.hpp:366-369 (launch_dense_mma_fp4_gate_up_bf16): gate and up of that segment in one
 * launch; the bits of two dgpp_launch_dense_mma_fp4_prod_bf16 calls. */
int dgpp_launch_dense_mma_fp4_gate_up_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* seg,
                                           const DgppMoeExpertView* views, uint16_t* gate, uint16_t* up, int m, int n,
                                           int k, void* stream, int fp4_group);
/* Extension (no counterpart in the reference): dgpp_launch_moe_grouped_mma{,_fp4}_bf16 for which = 0 and which = 1
 * followed by dgpp_launch_moe_swiglu_clamp, in one launch: a block walks its rows of the segment's gate matrix, then
 * of its up matrix, against the same activation rows and stores SwiGLU(bf16(gate), bf16(up)). Same bits as the
 * three launches. out: [sum of segment rows, out_stride] bf16 activation rows. */
int dgpp_launch_moe_grouped_mma_gate_up_swiglu(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs,
                                               int n_segs, int max_rows, int rows_per_block,
                                               const DgppMoeExpertView* views, uint16_t* out, size_t out_stride,
                                               int n, int k, float limit, void* stream, const int32_t* act_rows);
int dgpp_launch_moe_grouped_mma_gate_up_swiglu_fp4(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs,
                                                   int n_segs, int max_rows, int rows_per_block,
                                                   const DgppMoeExpertView* views, uint16_t* out, size_t out_stride,
                                                   int n, int k, float limit, void* stream, const int32_t* act_rows,
                                                   int fp4_group);
int dgpp_launch_moe_grouped_mma_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                         int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                         uint16_t* out, size_t out_stride, int n, int k, void* stream,
                                         const int32_t* act_rows, int fp4_group, int tile_rows);
int dgpp_launch_moe_grouped_mma_fp4_f32(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                        int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                        float* out, size_t out_stride, int n, int k, void* stream, const int32_t* act_rows,
                                        int fp4_group, int tile_rows);

/* src/kernels/fp4_gemv.hpp:23-32. `w` is a HOST struct holding device pointers.
 * Dispatch between the vector-core GEMV (up to eight rows per pass over the weights) or the matrix-core form (16 rows
 * per pass), chosen by what was measured faster on this chip: more rows than one vector pass holds -> matrix core; five
 * to eight rows -> matrix core when a split-K workspace is there (then from three rows on for matrices of 48 M weights
 * and more) or, without one, when the matrix has 64 M weights and more (an unsplit matrix-core launch has one block per
 * 64 weight rows: too few to fill the chip for smaller matrices); otherwise the vector core.
 * (This signature carries no workspace.) The reference moves to its tensor-core form as m grows in the same way
 * (src/kernels/glm_moe_launch.hpp:363). The two forms sum in different fp32 orders: a row's bits depend on which form
 * its call takes (a function of m, n, k only); both are held to the same oracle tolerance. */
int dgpp_launch_fp4_gemv_bf16(const uint16_t* act, size_t act_row_stride_elems,
                              const DgppFp4Matrix* w, uint16_t* out, int m, int n, int k,
                              void* stream);
int dgpp_launch_fp4_gemv_f32(const uint16_t* act, size_t act_row_stride_elems,
                             const DgppFp4Matrix* w, float* out, int m, int n, int k, void* stream);
/* 1 when the core accepts the matrix, else 0. */
int dgpp_fp4_gemv_accepts(const DgppFp4Matrix* w);

/* ---- dense FP8 block-scaled projection GEMV ------------------------------------------------------------ */
/* src/kernels/scale_gemm.hpp:57-79. Dispatch (reference: src/kernels/scale_gemm.cu:296-339) between
 * the vector-core GEMV (up to eight rows per pass over the weights) or the matrix-core form (16 rows
 * per pass), chosen by what was measured faster on this chip: more rows than one vector pass holds -> matrix core; five
 * to eight rows -> matrix core when a split-K workspace is there (then from three rows on for matrices of 48 M weights
 * and more) or, without one, when the matrix has 64 M weights and more (an unsplit matrix-core launch has one block per
 * 64 weight rows: too few to fill the chip for smaller matrices); otherwise the vector core.
 * A positive mma_from_rows adds the calls with m >= mma_from_rows to the matrix-core side. `ws` / `ws_bytes` (nullable;
 * parts(k) * m * n floats) is the split-K workspace. Split and unsplit give the same bits; the two cores sum in
 * different fp32 orders (both held to the same oracle tolerance), so a row's bits depend on which form its call takes
 * (a function of m, n, k and of whether a workspace is given). last_row_only / compact_row compute one row and stay
 * on the vector core. */
int dgpp_launch_scale_gemm_bf16(const uint16_t* act, size_t act_row_stride_elems,
                                const uint8_t* w_payload, const float* w_scales, uint16_t* out,
                                int m, int n, int k, void* stream, size_t out_row_stride_elems,
                                int mma_from_rows, void* ws, size_t ws_bytes);
int dgpp_launch_scale_gemm_f32(const uint16_t* act, size_t act_row_stride_elems,
                               const uint8_t* w_payload, const float* w_scales, float* out, int m,
                               int n, int k, void* stream, size_t out_row_stride_elems,
                               int mma_from_rows, int last_row_only, void* ws, size_t ws_bytes,
                               int compact_row);
/* src/kernels/scale_gemm.hpp:140-149: the same on a stated scale grid, with the same dispatch (ws as above; decode_mma
 * and prefill_tile are the reference's tuning hints and are accepted unused). */
int dgpp_launch_scale_gemm_grid_bf16(const uint16_t* act, size_t act_row_stride_elems,
                                     const uint8_t* w_payload, const float* w_scales, uint16_t* out,
                                     int m, int n, int k, void* stream,
                                     size_t out_row_stride_elems, int rs, int cs, int decode_mma,
                                     void* ws, size_t ws_bytes, int prefill_tile);
int dgpp_launch_scale_gemm_grid_f32(const uint16_t* act, size_t act_row_stride_elems,
                                    const uint8_t* w_payload, const float* w_scales, float* out,
                                    int m, int n, int k, void* stream, size_t out_row_stride_elems,
                                    int rs, int cs, int decode_mma, void* ws, size_t ws_bytes,
                                    int prefill_tile);
/* src/kernels/scale_gemm.hpp:155-162: the scale grid as e8m0 bytes (MXFP8: rs = 0, cs = 5). */
int dgpp_launch_scale_gemm_grid_e8m0_bf16(const uint16_t* act, size_t act_row_stride_elems,
                                          const uint8_t* w_payload, const uint8_t* w_scales,
                                          uint16_t* out, int m, int n, int k, void* stream,
                                          size_t out_row_stride_elems, int rs, int cs, void* ws,
                                          size_t ws_bytes, int prefill_tile);
int dgpp_launch_scale_gemm_grid_e8m0_f32(const uint16_t* act, size_t act_row_stride_elems,
                                         const uint8_t* w_payload, const uint8_t* w_scales,
                                         float* out, int m, int n, int k, void* stream,
                                         size_t out_row_stride_elems, int rs, int cs, void* ws,
                                         size_t ws_bytes, int prefill_tile);
/* src/kernels/scale_gemm.hpp:173-180 (launch_scale_gemm_tile_*): the scale GEMM's tile form for many rows; here the
 * matrix-core dense form (16 activation rows per pass over the weights). out row stride n. */
int dgpp_launch_scale_gemm_tile_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                     const float* w_scales, uint16_t* out, int m, int n, int k, void* stream, int rs, int cs);
int dgpp_launch_scale_gemm_tile_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                    const float* w_scales, float* out, int m, int n, int k, void* stream, int rs, int cs);
/* src/kernels/scale_gemm.hpp:85-107: up to four [n_i, k] fp8 matrices against the same rows, ONE launch (the grid is the
 * problems' row tiles laid end to end); each output is bitwise the single launcher's.
 * `problems` is a HOST array. bf16_weight must be null (that form is outside this path). */
typedef struct DgppFp8GemvProblem {
  const uint8_t* payload;
  const float* scales;
  uint16_t* out;
  int32_t n;
  int32_t reserved0;
  size_t out_stride;
  int32_t rs;
  int32_t cs;
  const uint16_t* bf16_weight;
} DgppFp8GemvProblem;
int dgpp_launch_scale_gemv_multi_bf16(const DgppFp8GemvProblem* problems, int n_problems,
                                      const uint16_t* act, size_t act_row_stride_elems, int rows,
                                      int k, void* stream);
/* src/kernels/scale_gemm.hpp:171: 1 when the fp8 GEMV can stage this payload at one row. */
int dgpp_fp8_gemv_can_stage(const void* w_payload, int k);

/* ---- FP8 -> BF16 dequant bridge ---------------------------------------------------------------------------- */
/* src/kernels/fp8_dequant.hpp:22-29 */
int dgpp_launch_fp8_dequant_blocks(const uint8_t* payload, const float* scales, uint16_t* out_bf16,
                                   int64_t rows, int64_t cols, void* stream, int rs, int cs);
int dgpp_launch_fp8_dequant_blocks_e8m0(const uint8_t* payload, const uint8_t* scales,
                                        uint16_t* out_bf16, int64_t rows, int64_t cols,
                                        void* stream, int rs, int cs);

/* ---- activation-quantized NVFP4 (W4A4) form ---------------------------------------------------------------------
 * The NVFP4 experts meet activations quantized to NVFP4 on the fly (per row a fp32 global gs, per 16 elements an e4m3
 * scale, e2m1 codes: x ~= e2m1 * scale * gs). Its numerics are those of src/kernels/moe_w4a4.cu, not of the
 * BF16-activation launchers above: the activations carry NVFP4 rounding. The quantizers reproduce the reference's
 * recipe bit for bit (a chain of single IEEE fp32 operations). The GEMM multiplies the exactly decoded operands on the
 * FP16 matrix core with FP32 accumulation (this chip's block-scaled FP4 instruction takes one power-of-two scale per 32
 * elements; NVFP4 carries an e4m3 per 16) and is held, like the reference's kernel, to the fp64 dot of the same
 * quantized operands: |got - dot| < 1e-5 * sum |terms| (tests/cuda/moe_w4a4_test.cu:193-216). */
/* src/kernels/moe_w4a4.hpp:15, moe_w4a4.cu:596: the activation scale buffer's row stride in bytes: k / 16 rounded up to 8. */
size_t dgpp_nvfp4_act_scale_stride(int k);
/* src/kernels/moe_w4a4.hpp:17-26, moe_w4a4.cu:598-611: BF16 rows [rows, k] (stride x_stride elements, a multiple of 8;
 * 16-byte aligned) -> codes [rows, k / 2] (low nibble = even element; 8-byte aligned), scales [rows,
 * dgpp_nvfp4_act_scale_stride(k)], gs [rows]. The global is *static_gs_dev when that DEVICE pointer is given, else
 * static_gs; a global <= 0 means amax / (6 * 448) per row (1 for a zero row); what exceeds 6 * 448 * gs saturates.
 * k a multiple of 64, <= 32768. */
int dgpp_launch_quantize_rows_nvfp4(const uint16_t* x, size_t x_stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                    float* gs, void* stream, float static_gs, const float* static_gs_dev);
/* src/kernels/moe_w4a4.hpp:27-35, moe_w4a4.cu:613-634: the same with the activation computed on the way - the MoE's
 * SwiGLU of (gate, up) with its clamp and two BF16 roundings (dgpp_launch_moe_swiglu_clamp's arithmetic), or with
 * qwen_rounding != 0 the dense MLP's of the Qwen family (silu as g / (1 + exp(-g)), one rounding of the product, no
 * clamp) - bitwise the activation kernel followed by the quantizer. */
int dgpp_launch_swiglu_quantize_rows_nvfp4(const uint16_t* gate, const uint16_t* up, size_t stride, int rows, int k,
                                           float limit, uint8_t* codes, uint8_t* scales, float* gs, void* stream,
                                           float static_gs, const float* static_gs_dev, int qwen_rounding);
/* src/kernels/moe_w4a4.hpp:37-49, moe_w4a4.cu:636-715: out[seg.row0 + m, :n] = act(row) . W(expert, which)^T for every
 * segment, act(row) the quantized row act_rows[seg.row0 + m] (or seg.row0 + m when act_rows is null); out = acc *
 * (gs[row] * (1 / global)). Segment / view / out conventions of dgpp_launch_moe_grouped_mma_fp4_*; k a multiple of 64. */
int dgpp_launch_moe_grouped_w4a4_bf16(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                                      const DgppMoeSegment* segs, int n_segs, int max_rows, const DgppMoeExpertView* views,
                                      int which, uint16_t* out, size_t out_stride, int n, int k, void* stream);
int dgpp_launch_moe_grouped_w4a4_f32(const uint8_t* codes, const uint8_t* scales, const float* gs, const int32_t* act_rows,
                                     const DgppMoeSegment* segs, int n_segs, int max_rows, const DgppMoeExpertView* views,
                                     int which, float* out, size_t out_stride, int n, int k, void* stream);

/* src/kernels/moe_w4a4.hpp:51-71 (dense_w4a4_tma_supported, launch_dense_w4a4_tma_bf16): the dense W4A4 form,
 * out[m, :n] = act(row) . W^T. The reference stages both code matrices through TMA tensor maps (nvfp4_code_tma_map);
 * this chip has no such descriptor, so the code matrices arrive as plain pointers ([m, k / 2] and [n, k / 2] bytes,
 * 16-byte aligned) and the map constructor has no counterpart. a_scales [m, a_scale_stride] and a_gs [m] are the
 * quantizer's, w_scales [n, k / 16] e4m3, w_global the matrix's device F32 global. k a multiple of 128. Bitwise the
 * grouped kernel over one segment, as in the reference. */
int dgpp_dense_w4a4_supported(int k);
int dgpp_launch_dense_w4a4_bf16(const uint8_t* a_codes, const uint8_t* a_scales, size_t a_scale_stride, const float* a_gs,
                                const uint8_t* w_codes, const uint8_t* w_scales, const float* w_global, uint16_t* out,
                                size_t out_stride, int m, int n, int k, void* stream);
/* src/kernels/minimax_native_moe.hpp:8-13, minimax_native_moe.cu:36-85, :97-107: the per-token dynamic NVFP4 producer of
 * the native routed experts: BF16 rows [rows, k] (any stride >= k) -> codes [rows, k / 2], e4m3 scales [rows, k / 16]
 * (dense, no padding), FP32 decode globals [rows] (amax / 2688; 0 for a zero row). Its scale chain multiplies by
 * reciprocals (see dgpp_amd/csrc/nvfp4_act.hip); they are the correctly rounded ones here, where the reference takes
 * NVIDIA's approximate reciprocal instruction: a scale byte or a code can differ from the reference's where that
 * instruction's last bit moves a rounding. k a multiple of 128, <= 32768. */
int dgpp_minimax_quantize_rows_nvfp4(const uint16_t* input, size_t stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                     float* globals, void* stream);
/* src/kernels/minimax_native_moe.hpp:15-18, minimax_native_moe.cu:87-95, :109-115: FP32 gate / up sums [count] ->
 * bf16((g' / (1 + exp(-alpha g'))) (u' + 1)), g' = min(g, limit), u' = clamp(u, -limit, limit). */
int dgpp_minimax_swiglu_f32(const float* gate, const float* up, uint16_t* output, int64_t count, float alpha, float limit,
                            void* stream);

/* ---- activation-quantized MXFP8 (W8A8) form ---------------------------------------------------------------------
 * The weights' MXFP8 payload meets activations quantized to MXFP8 on the fly; the products run on the
 * block-scaled matrix-core instruction (V_MFMA_SCALE_F32_16X16X128_F8F6F4, e8m0 scale per 32 values of
 * either operand), FP32 accumulation. Its numerics are those of src/kernels/mxfp8_gemm.cu, not of the
 * BF16-activation launchers above: the activations carry MXFP8 rounding.
 *
 * src/kernels/mxfp8_gemm.hpp:8-12, src/kernels/mxfp8_gemm.cu:246-256: BF16 x [rows, k] (row stride
 * x_stride elements) -> E4M3 codes [rows, k] and e8m0 scales [rows, k / 32]. A group's scale is
 * 2^ceil(log2(amax / 448)) (at least 2^-127; a zero group stores byte 0 and zero codes), its codes
 * e4m3_rne(x / scale). DGPP_INVALID_ARGUMENT unless k is a positive multiple of 32 and x_stride is at
 * least k and a multiple of 4; x must be 8-byte and codes 4-byte aligned; at most 65535 rows. */
int dgpp_launch_mxfp8_quantize_rows(const uint16_t* x, size_t x_stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                    void* stream);
/* src/kernels/mxfp8_gemm.hpp:14-18, src/kernels/mxfp8_gemm.cu:258-268: the same quantizer behind the clamped
 * SwiGLU of the MiniMax dense/shared MLP, v = bf16(g' * sigmoid(alpha * g') * (u' + 1)) with g' = min(g, limit),
 * u' = clamp(u, -limit, limit); sigmoid = 1 / (1 + 2^(-alpha * g' * log2 e)) through the hardware's
 * exponential and reciprocal. gate and up share `stride`. */
int dgpp_launch_minimax_swiglu_mxfp8_rows(const uint16_t* gate, const uint16_t* up, size_t stride, int rows, int k, float alpha,
                                          float limit, uint8_t* codes, uint8_t* scales, void* stream);
/* src/kernels/mxfp8_gemm.hpp:20-31, src/kernels/mxfp8_gemm.cu:217-243, :270-279: out[m, n] = A[m, k] * W[n, k]^T,
 * both operands row-major E4M3 with e8m0 scales [rows, k / 32]; out_stride in output elements (0 -> n).
 * DGPP_INVALID_ARGUMENT unless k is a positive multiple of 64, out_stride >= n and output_tile is one of
 * 0, 8, 16, 32, 64 (a diagnostic of the reference's kernel: accepted, and without effect here); both payloads
 * 16-byte aligned. An output element's value depends on its own two rows and k only, never on m, n or
 * the rows sharing the launch; the bf16 form is the f32 form rounded to nearest even. */
int dgpp_launch_mxfp8_gemm_bf16(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales,
                                uint16_t* out, int m, int n, int k, void* stream, size_t out_stride, int output_tile);
int dgpp_launch_mxfp8_gemm_f32(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales, float* out,
                               int m, int n, int k, void* stream, size_t out_stride, int output_tile);

/* ---- the gated shared expert's decode tail, block-FP8 weights -------------------------------------------------
 * src/kernels/qwen_moe.hpp:12-19, src/kernels/qwen_moe.cu:312-326: w[t] = bf16(sigmoid(bf16(x[t] . g))) as an F32
 * value; x BF16 [tokens, hidden] (dense rows), g BF16 [hidden] or NULL (then w[t] = 1). The dot runs in the
 * reference's order: 32 strided partial sums over 16-byte vectors and the xor tree 16, 8, 4, 2, 1.
 * DGPP_INVALID_ARGUMENT unless hidden is a positive multiple of 8 and x, g are 16-byte aligned. */
int dgpp_qwen_moe_shared_gate_bf16(const uint16_t* x, const uint16_t* g, float* w, int tokens, int hidden, void* stream);
/* src/kernels/qwen_moe.hpp:34-87, the FP8 forms (src/kernels/qwen_moe.cu:377-413, :443-482). The tail in two launches:
 *   gate_up:  act[t, s] = swiglu(bf16(x[t] . gate[s]), bf16(x[t] . up[s])) without clamps, BF16 [tokens, S];
 *             sw[t] as dgpp_qwen_moe_shared_gate_bf16 (x rows at x_stride);
 *   down:     out[t, h] = bf16(fma(sw[t], act[t] . down[h], a)), a = acc[t, h] (F32 [tokens, H]), or, in the
 *             routed form, the fma chain over j < top_k of weights[t, j] * contrib[(t * (top_k + 1) + j), h]
 *             from zero (the routed accumulate kernel's order), top_k <= 16.
 * gate / up: E4M3 [S, H], down: E4M3 [H, S], F32 scales on the (rs, cs) grid (log2 block rows / columns, cs >= 4).
 * tokens <= 8 (one pass over the weights for all of them), H and S multiples of 16, operands 16-byte aligned.
 * Each launch is bitwise the unfused launchers it stands for (dgpp_launch_scale_gemm_grid_bf16 twice,
 * dgpp_launch_moe_swiglu_clamp with an infinite limit, dgpp_launch_scale_gemm_grid_f32, the gate, the accumulate,
 * dgpp_launch_moe_round_bf16). The halves are entries of their own so that gate_up can run beside the routed
 * experts on another stream; the BF16-weight forms of the reference's tail are not provided. */
int dgpp_qwen_moe_shared_gate_up_decode_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                            const uint8_t* up_p, const float* up_s, const uint16_t* g, uint16_t* act, float* sw,
                                            int tokens, int H, int S, void* stream, int rs, int cs);
int dgpp_qwen_moe_shared_down_decode_fp8(const uint16_t* act, const uint8_t* down_p, const float* down_s, const float* sw,
                                         const float* acc, uint16_t* out, int tokens, int H, int S, void* stream, int rs,
                                         int cs);
int dgpp_qwen_moe_shared_down_decode_routed_fp8(const uint16_t* act, const uint8_t* down_p, const float* down_s, const float* sw,
                                                const float* contrib, const float* weights, int top_k, uint16_t* out,
                                                int tokens, int H, int S, void* stream, int rs, int cs);
int dgpp_qwen_moe_shared_tail_decode_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                         const uint8_t* up_p, const float* up_s, const uint8_t* down_p, const float* down_s,
                                         const uint16_t* g, uint16_t* act, float* sw, const float* acc, uint16_t* out,
                                         int tokens, int H, int S, void* stream, int rs, int cs);
int dgpp_qwen_moe_shared_tail_decode_routed_fp8(const uint16_t* x, size_t x_stride, const uint8_t* gate_p, const float* gate_s,
                                                const uint8_t* up_p, const float* up_s, const uint8_t* down_p,
                                                const float* down_s, const uint16_t* g, uint16_t* act, float* sw,
                                                const float* contrib, const float* weights, int top_k, uint16_t* out,
                                                int tokens, int H, int S, void* stream, int rs, int cs);

/* ---- host-side weight encoders and synthetic data (no GPU involved) ------------------------------------------ */
/* Scalar codecs, src/common/dtypes.hpp:83-190, src/kernels/latent_format.hpp:117-162. */
float dgpp_bf16_to_f32(uint16_t bits);
uint16_t dgpp_f32_to_bf16(float v);
float dgpp_e4m3_to_f32(uint8_t code);
uint8_t dgpp_f32_to_e4m3(float v);
float dgpp_e2m1_to_f32(uint8_t code);
uint8_t dgpp_f32_to_e2m1(float v);
float dgpp_e8m0_to_f32(uint8_t code);
uint8_t dgpp_e8m0_ceil_log2(float v);
/* Block FP8 encoder, src/loaders/fp8_quant.hpp:32-46 generalised to any block size:
 * scale_b = amax/448 (zero block: 1), code = e4m3_rne_sat(w / scale_b). src bf16 [rows, cols]. */
void dgpp_encode_fp8_blocks(const uint16_t* src_bf16, int64_t rows, int64_t cols, int block_rows,
                            int block_cols, uint8_t* payload, float* scales, int threads);
/* NVFP4 encoder, src/loaders/nvfp4_quant.hpp:25-55. Returns weight_scale_2; the DEVICE global the
 * kernels divide by is 1 / weight_scale_2. src f32 [rows, cols], cols % 16 == 0. */
float dgpp_encode_nvfp4(const float* src, int64_t rows, int64_t cols, uint8_t* payload,
                        uint8_t* scales, int threads);
/* MXFP4 / MXFP8 encoders: one e8m0 byte per 32 elements chosen by the reference's own e8m0
 * producers' rule, b = 127 + ceil(log2(amax / fmt_max)) from the IEEE fields
 * (src/kernels/latent_format.hpp:117-123, src/kernels/mxfp8_gemm.cu:61-66), codes RNE saturating;
 * an all-zero block stores byte 0 and zero codes. src f32 [rows, cols], cols % 32 == 0. */
void dgpp_encode_mxfp4(const float* src, int64_t rows, int64_t cols, uint8_t* payload,
                       uint8_t* scales, int threads);
void dgpp_encode_mxfp8(const float* src, int64_t rows, int64_t cols, uint8_t* payload,
                       uint8_t* scales, int threads);
/* Seeded synthetic data: xorshift64 (tests/cuda/scale_gemm_test_helpers.hpp:29-47's generator
 * family) + Box-Muller; element i of a stream depends on (seed, i / 4096) only, so the output does
 * not depend on `threads`. */
void dgpp_fill_normal_f32(uint64_t seed, float mean, float stddev, int64_t n, float* out,
                          int threads);
void dgpp_fill_normal_bf16(uint64_t seed, float mean, float stddev, int64_t n, uint16_t* out,
                           int threads);
/* top_k distinct expert ids per token drawn without replacement from Zipf(s) popularity over
 * n_experts (expert e has weight 1/(e+1)^s), ids ascending per token. */
void dgpp_fill_zipf_routes(uint64_t seed, double s, int tokens, int top_k, int n_experts,
                           int32_t* ids);

#ifdef __cplusplus
}
#endif
#endif /* DGPP_AMD_H */
