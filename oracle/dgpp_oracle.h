/*
 * CPU oracle for the quantized MoE expert GEMV path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain host restatement of the reference's
 * algorithms for the path (codecs, dequantisation, fp64 dot products, router
 * selection, token->expert grouping, SwiGLU, ordered accumulation). It is what
 * the HIP kernels are checked against and what the benchmark times as the CPU
 * baseline. Product code must never call into it.
 *
 * Each function names the reference file:line it restates (paths relative to the
 * reference's repository root).
 *
 * How every function here is pinned (none is "parity unpinned"):
 *   codecs            exhaustive tables + the reference's own unit-test KATs + the
 *                     compiled reference (oracle/_ref) over every code / a float sweep
 *   dequant / gemv    brute-force numpy fp64 on small shapes + oracle/_ref forward
 *   router select     compiled reference router + all-equal-scores closed form
 *   grouping/order    brute-force stable sort in numpy + permutation invariants
 *   swiglu            compiled reference forward (I = 1 degenerate chain) + edge KATs
 *   accumulation      numpy float32 fma emulation through float64 (exact for one fma)
 *   moe forward       compiled reference glm_moe_ref_forward, FP8 / NVFP4 / MXFP4
 *   mxfp8 quantizer   the closed form of the reference's own kernel test in numpy float64, all finite BF16
 *   mxfp8 gemm        numpy float64 brute force; swiglu-oai: closed-form points + numpy
 */
#ifndef DGPP_ORACLE_H
#define DGPP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar codecs -------------------------------------------------------- */
/* src/common/dtypes.hpp:83-100 */
float orc_bf16_to_f32(uint16_t bits);
uint16_t orc_f32_to_bf16(float v);
/* src/common/dtypes.hpp:135-190 (OCP E4M3FN, saturating RNE encode) */
float orc_e4m3_to_f32(uint8_t code);
uint8_t orc_f32_to_e4m3(float v);
/* src/kernels/latent_format.hpp:134-162 */
float orc_e2m1_to_f32(uint8_t code);
uint8_t orc_f32_to_e2m1(float v);
/* src/kernels/latent_format.hpp:117-128 */
float orc_e8m0_to_f32(uint8_t code);
uint8_t orc_e8m0_ceil_log2(float v);

/* ---- dequantisation to double -------------------------------------------- */
/* FP8 block-scaled weights: w = bf16_rne(float(e4m3) * scale) when strict != 0
 * (src/models/glm/moe_reference.cpp:160-173, src/kernels/fp8_gemv.cuh:64-66),
 * the exact product in double otherwise (tests/cuda/scale_gemm_test_helpers.hpp:118-136).
 * Exactly one of scales_f32 / scales_e8m0 is non-null; the grid is
 * [ceil(rows/2^rs), ceil(cols/2^cs)] row-major. An e8m0 byte b stands for the float
 * whose exponent field is b (0 -> 2^-127), src/kernels/fp8_dequant.cu:28-31. */
void orc_dequant_fp8(const uint8_t* payload, const float* scales_f32, const uint8_t* scales_e8m0,
                     int64_t rows, int64_t cols, int rs, int cs, int strict, double* out);
/* FP4 weights without the global scale: e2m1(code) * e4m3(scale) (group 16) or
 * e2m1(code) * 2^(b-127) (group 32, b == 255 -> NaN).
 * src/models/glm/moe_reference.cpp:78-94 */
void orc_dequant_fp4(const uint8_t* payload, const uint8_t* scales, int group, int64_t rows,
                     int64_t cols, double* out);

/* ---- single-matrix GEMV oracles: out_raw[m, n] in double, unrounded ------- */
/* src/models/glm/moe_reference.cpp:37-72; tests/cuda/scale_gemm_test_helpers.hpp:107-142 */
void orc_gemv_fp8(const uint16_t* act, int64_t act_stride, const uint8_t* payload,
                  const float* scales_f32, const uint8_t* scales_e8m0, int m, int n, int k, int rs,
                  int cs, int strict, double* out_raw);
/* divisor = the NVFP4 device global (the finished dot is divided by it), 1 for MXFP4.
 * src/models/glm/moe_reference.cpp:37-52 with 78-94 */
void orc_gemv_fp4(const uint16_t* act, int64_t act_stride, const uint8_t* payload,
                  const uint8_t* scales, double divisor, int group, int m, int n, int k,
                  double* out_raw);

/* ---- router --------------------------------------------------------------- */
enum { ORC_ROUTER_SIGMOID = 0, ORC_ROUTER_SOFTMAX = 1, ORC_ROUTER_SQRT_SOFTPLUS = 2 };
/* hidden bf16 [tokens, hidden], gate bf16 [experts, hidden], bias f32 [experts] (null in
 * softmax mode) -> scores/biased [tokens, experts] in double. Softmax mode leaves the
 * bf16-rounded logit in both. src/models/glm/moe_reference.cpp:295-317 */
void orc_router_scores(const uint16_t* hidden, const uint16_t* gate, const float* bias, int mode,
                       int tokens, int experts, int hidden_dim, double* scores, double* biased);
/* top-k on biased (strict >, lower id wins ties), ids ascending, weights
 * w/(sum + 1e-20) * scale (softmax: probabilities of the full row, result rounded to bf16).
 * src/models/glm/moe_reference.cpp:318-366 */
void orc_router_select(const double* scores, const double* biased, int mode, int tokens,
                       int experts, int top_k, double scaling, int norm_topk, int32_t* ids,
                       float* weights);

/* ---- grouping (all integer, bit-exact contracts) --------------------------- */
/* Host counting sort: rows[pos] = token for every (token, slot) ordered by ascending expert,
 * stable in (token, slot); slot_row[t*K+j] = pos; segs[e] = {row0, rows, e} for every expert,
 * segs[E] = {T*K, T, E}; rows[T*K + t] = t. segs is int32 [E+1][3].
 * src/models/glm/moe_layer.cpp:634-659; src/kernels/glm_moe.cu:1382-1439 */
void orc_moe_segment(const int32_t* ids, int tokens, int top_k, int experts, int32_t* rows,
                     int32_t* slot_row, int32_t* segs);
/* Slot execution order over tokens*(K+1) slots keyed by expert id (shared = experts), stable;
 * optional shared_early remap; optional runs[slots + slots/17 + 1].
 * src/kernels/glm_moe.cu:465-517 */
void orc_moe_slot_order(const int32_t* ids, int slots, int top_k, int experts, int shared_early,
                        int32_t* order, int32_t* runs);
/* tiles[i] = {seg, m0} in segment order; returns the count. src/kernels/glm_moe.cu:1553-1569 */
int orc_moe_tile_list(const int32_t* segs, int n_segs, int tile_rows, int32_t* tiles);
/* Stable compaction of non-empty segments into `capacity` entries, the rest zeroed.
 * src/kernels/minimax.cu:33-50 */
void orc_compact_segments(const int32_t* segs_in, int32_t* segs_out, int experts, int capacity);

/* ---- elementwise pieces ----------------------------------------------------- */
/* act = bf16(bf16(g*sigmoid(g)) * u), g clamped above only, u both sides; math in double.
 * src/models/glm/moe_reference.cpp:176-189 */
void orc_swiglu(const uint16_t* gate, const uint16_t* up, int64_t n, float limit, uint16_t* out);
/* The fp32 fmaf chains, bitwise contracts.
 * src/kernels/glm_moe.cu:673-711 (slot layout), :1446-1489 (ordered/grouped layout), :371-393 */
void orc_slot_accum(const float* contrib, const float* weights, int tokens, int hidden, int top_k,
                    int with_shared, float* out_f32, uint16_t* out_bf16);
void orc_accum_ordered(const float* down, int64_t down_stride, const int32_t* slot_row,
                       const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                       int top_k, int hidden, float* out_f32, uint16_t* out_bf16);

/* ---- full MoE layer oracle ---------------------------------------------------- */
/* One expert matrix in any of the path's formats. */
typedef struct {
  const uint8_t* payload;     /* fp8: [rows, cols]; fp4: [rows, cols/2] */
  const float* scales_f32;    /* fp8 F32 grid, else null */
  const uint8_t* scales_u8;   /* fp8 e8m0 grid, or fp4 scales */
  double divisor;             /* NVFP4 device global (dot is divided by it); else 1 */
  int32_t kind;               /* 0 fp8, 1 fp4 */
  int32_t group;              /* fp4: 16 or 32 */
  int32_t rs, cs;             /* fp8 scale grid log2 block sizes */
} OrcMatrix;

/* Strict layer oracle over given routes: per token, experts ascending, gate/up dots in fp64
 * rounded to bf16, SwiGLU, down dots unrounded, acc += w * down, then (optional) the shared
 * expert with weight 1, one bf16 rounding. experts = [n_experts*3] gate,up,down; shared = [3]
 * or null. out_raw (double, unrounded, nullable) and out_bf16 (nullable) are [tokens, hidden].
 * threads > 1 spreads weight rows over std::thread workers (same arithmetic per element).
 * src/models/glm/moe_reference.cpp:369-468; src/models/qwen/moe_reference.cpp:119-160 */
void orc_moe_forward(const uint16_t* x, int64_t x_stride, const int32_t* ids, const float* weights,
                     int tokens, int top_k, int hidden, int inter, int shared_inter,
                     const OrcMatrix* experts, const OrcMatrix* shared, float swiglu_limit,
                     int threads, double* out_raw, uint16_t* out_bf16);

/* The gated shared expert's weight: w[t] = bf16(sigmoid(bf16(x[t] . g))) with the dot and the sigmoid in double
 * (g null: 1). src/models/qwen/moe_reference.cpp:153-157. Pinned by numpy float64 and closed-form points
 * (x = 0 -> 0.5; a large logit -> 1). */
void orc_shared_gate(const uint16_t* x, int64_t x_stride, const uint16_t* g, int tokens, int hidden, float* w);

/* ---- activation-quantized MXFP8 form (its own numerics contract: the activations carry MXFP8 rounding) ---- */
/* BF16 x [rows, k] (row stride in elements) -> E4M3 codes [rows, k], e8m0 scales [rows, k / 32]: per
 * 32-group the exponent is max(-127, ceil(log2(amax / 448))) (a zero group: -127, byte 0), codes are
 * e4m3_rne_sat(x * 2^-exponent). src/kernels/mxfp8_gemm.cu:58-79.
 * Pinned by the closed form the reference's own test checks its kernel with, evaluated in numpy float64
 * (ceil(log2(amax / 448)), tests/cuda/mxfp8_gemm_test.cu:77-92) over every finite BF16 pattern and the
 * 446 / 448 / 450 * 2^e boundary rows of that test (:96-123); the code conversion is orc_f32_to_e4m3. */
void orc_mxfp8_quantize_rows(const uint16_t* x, int64_t stride, int rows, int k, uint8_t* codes, uint8_t* scales);
/* The clamped SwiGLU the fused quantizer applies first, in double:
 * min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, +-limit) + 1); `exact` (nullable) unrounded,
 * `rounded` (nullable) as BF16, both [rows, k] dense. src/kernels/mxfp8_gemm.cu:37-56 states the formula,
 * tests/cuda/mxfp8_gemm_test.cu:155-170 the double form used here. Pinned by closed-form points
 * (g = 0, u = -1, saturated clamps) and numpy. */
void orc_swiglu_oai(const uint16_t* gate, const uint16_t* up, int64_t stride, int rows, int k, float alpha, float limit,
                    double* exact, uint16_t* rounded);
/* out[m, n] = sum_k e4m3(a) 2^(sa - 127) * e4m3(w) 2^(sw - 127) in double, and (nullable) the same sum of
 * magnitudes for the forward-error bound. tests/cuda/mxfp8_gemm_test.cu:222-236. Pinned by numpy brute force. */
void orc_mxfp8_gemm(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales, int m, int n, int k,
                    double* out, double* out_abs);

/* ---- activation-quantized NVFP4 form (W4A4: the activations carry NVFP4 rounding) ---- */
/* BF16 x [rows, k] (row stride in elements) -> e2m1 codes [rows, k / 2] (low nibble = even element), e4m3 block scales
 * [rows, scale_stride] (one per 16 elements), gs[rows]: x ~= e2m1 * scale * gs. The row's global is static_gs when > 0
 * (what exceeds 6 * 448 * gs saturates), else amax / (6 * 448) (1 for a zero row); a block's scale is
 * e4m3_rne_sat(amax16 / (6 * gs)); codes are e2m1_rne_sat(x * (1 / (scale * gs))); a zero block or a zero scale
 * gives scale byte 0 and codes 0. Every operation is a single IEEE fp32 operation in the reference
 * (src/kernels/moe_w4a4.cu:139-236), so the restatement is bit-exact by construction.
 * Pinned by the reference test's known-answer rows (values representable under scale 0.25 and a static global of 1 come
 * back bit for bit, tests/cuda/moe_w4a4_test.cu:291-326), closed-form points (zero rows, saturation at 6 * 448 * gs)
 * and an independent numpy float32 evaluation of the same recipe; the conversions are orc_f32_to_e4m3 / orc_f32_to_e2m1. */
void orc_nvfp4_quantize_rows(const uint16_t* x, int64_t stride, int rows, int k, float static_gs, uint8_t* codes,
                             uint8_t* scales, int64_t scale_stride, float* gs);
/* src/kernels/glm_moe.cu:917-949 (hash routing): ids[t] = row tokens[t] of tid2eid (row 0 for a token outside the
 * vocabulary), weights = scores at those ids, / (their fp32 sum in row order + 1e-20) when norm_topk, * scaling.
 * Pinned by an independent numpy float32 evaluation (cumulative sums in float32) and closed-form rows. */
void orc_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int n_tokens, int vocab,
                     int n_experts, int top_k, float scaling, int norm_topk, int32_t* ids, float* weights);
/* The per-token dynamic NVFP4 producer of src/kernels/minimax_native_moe.cu:36-85: scales [rows, k / 16] (dense),
 * globals[rows] = amax * (1 / 2688) (0 for a zero row). The chain of fp32 multiplications by reciprocals is restated
 * with every reciprocal correctly rounded. PARITY UNPINNED against the reference in that one respect: its reciprocal is
 * NVIDIA's approximate instruction (rcp.approx.ftz.f32), whose last bit no fixture or closed form available here
 * fixes (the reference's own test reads fixture folders that are not in its tree). What IS pinned: the restated chain
 * against an independent numpy float32 evaluation, the decode identity (decoded rows within half a code step), zero
 * rows, and invariance to how rows are spread over calls (the property the reference's test checks). */
void orc_minimax_quantize_rows_nvfp4(const uint16_t* x, int64_t stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                     float* globals);
/* The MiniMax router: selection and weights from sigmoid scores, FP32 throughout (ranking by score + bias, ties to
 * the lower id, ids ascending, weights = score / max(sum in id order, 1e-20) * factor).
 * src/models/minimax/reference.cpp:96-113; src/kernels/minimax.cu:409-440 */
void orc_minimax_route_scores(const float* scores, const float* bias, int rows, int experts, int topk, float factor,
                              int32_t* ids, float* weights);
/* scores[r, e] = sigmoid(dot(x[r], gate[e])), dot in double; x BF16 bits, gate FP32. src/kernels/minimax.cu:397-408 */
void orc_minimax_router_scores(const uint16_t* x, const float* gate, int rows, int hidden, int experts, double* scores);
/* src/kernels/minimax_native_moe.cu:87-95 evaluated in double: bf16((g' / (1 + exp(-alpha g'))) (u' + 1)), g' = min(g,
 * limit), u' = clamp(u, -limit, limit); out (nullable) the BF16 rounding, out_exact (nullable) the unrounded value.
 * Pinned by closed-form points (g = 0, u = -1, both clamps) and numpy float64. */
void orc_minimax_swiglu_f32(const float* gate, const float* up, int64_t count, double alpha, double limit, uint16_t* out,
                            double* out_exact);
/* out[m, n] = (sum_k e2m1(a) e4m3(sa) * e2m1(w) e4m3(sw)) * gs[m] / w_global in double, and (nullable) the same sum of
 * magnitudes: the fp64 dot of the SAME quantized operands the reference's kernel test compares against
 * (tests/cuda/moe_w4a4_test.cu:193-216, bound |got - dot| < 1e-5 * sum|terms|). Pinned by numpy brute force. */
void orc_w4a4_gemm(const uint8_t* a_codes, const uint8_t* a_scales, int64_t a_scale_stride, const float* a_gs,
                   const uint8_t* w_codes, const uint8_t* w_scales, double w_global, int m, int n, int k, double* out,
                   double* out_abs);

/* ---- comparators ---------------------------------------------------------------- */
typedef struct {
  double l2_rel;
  double max_rel;       /* max |got - oracle| / max(|oracle|, floor_abs) */
  double max_ulps;      /* max |got - oracle| / bf16_ulp(oracle) among elements above the floor */
  int64_t mismatches;   /* elements beyond BOTH ulp_budget ulps and the absolute floor */
  int64_t nan_pattern_errors;
  int64_t total;
} OrcCompare;
/* tests/cuda/scale_gemm_test_helpers.hpp:53-100: an element fails when |diff| exceeds both
 * ulp_budget bf16 ulps at the oracle's magnitude and floor_frac * max|oracle|. */
void orc_compare_bf16(const uint16_t* got, const double* oracle, int64_t n, double ulp_budget,
                      double floor_frac, OrcCompare* rep);
void orc_compare_f32(const float* got, const double* oracle, int64_t n, double ulp_budget,
                     double floor_frac, OrcCompare* rep);

#ifdef __cplusplus
}
#endif
#endif
