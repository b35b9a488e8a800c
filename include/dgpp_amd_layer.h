/*
 * C entry points of the host-side MoE layer driver (dgpp_amd/csrc/moe_layer.{hpp,cpp}): the
 * counterpart of the reference's GlmMoeLayer (src/models/glm/moe_layer.hpp:50, call order of
 * enqueue_decode_impl at src/models/glm/moe_layer.cpp:1415-1680 and of the device-segmented grouped
 * path at :775-817, :906-934). The driver is C++ above the kernel ABI of dgpp_amd.h; these wrappers
 * let tests and the benchmark drive it through ctypes. Unlike the launchers, create / destroy
 * allocate and free device memory (the layer's scratch and its device expert table).
 */
#ifndef DGPP_AMD_LAYER_H
#define DGPP_AMD_LAYER_H

#include "dgpp_amd.h"
#include "dgpp_amd_loader.h"

#ifdef __cplusplus
extern "C" {
#endif

#define DGPP_EXPERTS_FP8 0
#define DGPP_EXPERTS_NVFP4 1
#define DGPP_EXPERTS_MXFP4 2

typedef struct DgppMoeLayer DgppMoeLayer;
/* Message of the calling thread's last failed layer call. */
const char* dgpp_moe_layer_last_error(void);

typedef struct DgppMoeLayerDesc {
  DgppMoeConfig cfg;
  int32_t expert_format;              /* DGPP_EXPERTS_* */
  int32_t max_tokens;
  const DgppMoeExpertView* views;     /* HOST array: [n_experts * 3] gate,up,down, then the shared
                                         triple when shared_in_table != 0 */
  int32_t shared_in_table;            /* the shared expert is an FP4 triple at views[n_experts * 3 ..] */
  int32_t shared_inter;               /* the shared expert's intermediate width (0: no shared expert) */
  const uint8_t* sh_payload[3];       /* FP8 shared expert given as launch arguments (gate, up, down) */
  const float* sh_scales[3];
  int32_t sh_rs, sh_cs;
  const uint16_t* router_gate;        /* bf16 [n_experts, hidden] (may be null when only
                                         enqueue_decode_scores is used) */
  const float* router_bias;           /* f32 [n_experts] (null in softmax mode) */
  const uint8_t* sh_scales_e8m0[3];   /* all three non-null: the shared expert is an MXFP8 expert (E4M3 payload in
                                         sh_payload, one E8M0 scale byte per 32 columns here; sh_scales, sh_rs and sh_cs
                                         unused) of its OWN width shared_inter, run as dense projections over the
                                         batch's token rows beside the routed passes (reference:
                                         src/models/minimax/layers.cpp:34-45, 222-238) and added last to each token's
                                         chain with weight 1, one rounding. hidden and shared_inter multiples of 32. */
} DgppMoeLayerDesc;

/* Device bytes the layer's scratch takes for max_tokens (reference: GlmMoeLayer::scratch_bytes,
 * src/models/glm/moe_layer.cpp:72-129, decode-slot and grouped buffers). */
size_t dgpp_moe_layer_scratch_bytes(const DgppMoeConfig* cfg, int max_tokens, int shared_inter);
/* The same for a layer whose shared expert is the dense MXFP8 form (sh_scales_e8m0 given). */
size_t dgpp_moe_layer_scratch_bytes_dense_shared(const DgppMoeConfig* cfg, int max_tokens, int shared_inter);
int dgpp_moe_layer_create(const DgppMoeLayerDesc* desc, DgppMoeLayer** out);
void dgpp_moe_layer_destroy(DgppMoeLayer* layer);

/* The decode path: router -> slot order (tokens > 1) -> gate/up+SwiGLU -> down -> accumulate, all
 * on `stream`, no host sync. out_bf16 [tokens, hidden]; out_f32 (nullable) receives the unrounded
 * chain instead when given. x bf16 [tokens, x_stride]. */
int dgpp_moe_layer_enqueue_decode(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride, uint16_t* out_bf16,
                                  float* out_f32, int tokens, void* stream);
/* The same with the router's scores given (f32 [tokens, n_experts] scores and biased rows; softmax
 * mode: the bf16-rounded logits in both): only the selection half of the router runs. */
int dgpp_moe_layer_enqueue_decode_scores(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride,
                                         const float* scores, const float* biased, uint16_t* out_bf16,
                                         float* out_f32, int tokens, void* stream);
/* The same with the routes given (ids ascending per token, weights): no router at all. */
int dgpp_moe_layer_enqueue_decode_routed(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride,
                                         const int32_t* ids, const float* weights, uint16_t* out_bf16,
                                         float* out_f32, int tokens, void* stream);
/* The grouped (segment-major) path over given routes: device segmentation -> gather -> grouped
 * gate, up -> SwiGLU -> grouped down -> ordered accumulation. Bitwise the decode path's output. */
int dgpp_moe_layer_enqueue_grouped_routed(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride,
                                          const int32_t* ids, const float* weights, uint16_t* out_bf16,
                                          float* out_f32, int tokens, void* stream);
/* The grouped path through the matrix-core launchers (the reference's prefill form,
 * src/models/glm/moe_layer.cpp:775-817): gather folded into the gate / up launches. A layer's shared expert rides
 * along as the segment of every token behind the routed rows (:1293-1296, 1335-1336; a table entry joins the routed
 * launches, a block-FP8 one of its own width takes a launch of its own per projection) and ends every token's chain
 * with weight 1; the dense MXFP8 form runs beside the routed chain as in the decode path. */
int dgpp_moe_layer_enqueue_prefill_routed(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride, const int32_t* ids,
                                          const float* weights, uint16_t* out_bf16, float* out_f32, int tokens,
                                          void* stream);
/* The same from the hidden rows (GlmMoeLayer::enqueue_prefill, src/models/glm/moe_layer.cpp:775-812: routing stays on the
 * device, nothing waits on the host): score rows, selection, then the chain above over the layer's own ids and weights. */
int dgpp_moe_layer_enqueue_prefill(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride, uint16_t* out_bf16, float* out_f32,
                                   int tokens, void* stream);
/* The prefill in phases (route_prefill_rows / enqueue_prefill_phased / accumulate_prefill_rows,
 * src/models/glm/moe_layer.cpp:843-904), for a caller that overlaps other work with the per-row ends of the layer: the router
 * over rows [r0, r0 + rows) of x (x points at row 0), then the chain over all `tokens` rows without its accumulation, then
 * the accumulation of rows [r0, r0 + rows) into out[r0 ...] (out points at row 0). The same kernels per row as
 * dgpp_moe_layer_enqueue_prefill: bitwise its output. The shared expert rides as a segment (not the dense MXFP8 form). */
int dgpp_moe_layer_route_prefill_rows(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride, int r0, int rows, void* stream);
int dgpp_moe_layer_enqueue_prefill_phased(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride, int tokens, void* stream);
int dgpp_moe_layer_accumulate_prefill_rows(DgppMoeLayer* layer, uint16_t* out_bf16, float* out_f32, int tokens, int r0, int rows,
                                           void* stream);
/* The activation-quantized (W4A4) form of that chain for NVFP4 experts (src/models/glm/moe_layer.cpp:1122-1135,
 * 1217-1219, 1268-1272, 1306-1316): token rows -> NVFP4 row quantizer -> grouped W4A4 gate, up over the routed row list
 * -> SwiGLU inside the second quantizer -> grouped W4A4 down (bf16 rows, or f32 when f32_down is non-zero, the
 * reference's DGPP_MOE_W4A4_F32_DOWN) -> ordered accumulation. act_scales_dev: null for a global per row, or a
 * DEVICE pair {token rows' global, SwiGLU rows' global} (the reference's act_scales_dev). hidden and inter must
 * be multiples of 64. Bitwise the same launchers called one by one. A shared expert keeps BF16 activations: its
 * segment's rows sit behind the routed rows (then every down row is f32, :1121), the MXFP8 form runs beside. */
int dgpp_moe_layer_enqueue_prefill_routed_w4a4(DgppMoeLayer* layer, const uint16_t* x, size_t x_stride, const int32_t* ids,
                                               const float* weights, uint16_t* out_bf16, float* out_f32, int tokens,
                                               void* stream, const float* act_scales_dev, int f32_down);
/* Waits for `stream` and reports whether a decode call enqueued on it ended with its one-launch expert chain
 * (dgpp_launch_moe_slot_chain*) giving up the bounded wait for its gate/up rows: DGPP_RUNTIME_ERROR then (that
 * call's output is invalid; the layer's counters are back at rest), DGPP_OK otherwise. Synchronizes: not for
 * use under stream capture. No counterpart in the reference, whose launches wait for each other at launch
 * boundaries only. */
int dgpp_moe_layer_check(DgppMoeLayer* layer, void* stream);
/* Device pointers of the last routes the layer computed: ids int32 [tokens, top_k], weights f32. */
const DgppMoeExpertView* dgpp_moe_layer_views(const DgppMoeLayer* layer); /* the device expert table */
const int32_t* dgpp_moe_layer_ids(const DgppMoeLayer* layer);
const float* dgpp_moe_layer_weights(const DgppMoeLayer* layer);

/* ---- a bound layer made resident in one call -----------------------------------------------------------------
 * Reference: the resident build of a MoE layer, src/models/glm/loader.cpp:418-471 (router, shared expert, every
 * routed expert cut to the rank's slice of the intermediate dimension, NVFP4 globals gathered into one array), with
 * the slicing rules of src/models/quant_matrix.hpp:67-96 (block-FP8 grids re-blocked at gcd(128, start, count)) and
 * :140-164 (FP4 column slices on scale-group boundaries). Takes what a dgpp_*_moe_bind_layer call found (host
 * addresses inside the mapped shards, which must stay open during the call), uploads this rank's slices into ONE
 * device allocation and creates the layer driver over them. Not a launcher: it allocates, copies and synchronizes. */
typedef struct DgppMoeResident DgppMoeResident;
typedef struct DgppMoeResidentDesc {
  DgppMoeConfig cfg;                    /* the checkpoint's (unsliced) geometry */
  int32_t max_tokens;
  int32_t rank, world;                  /* gate / up rows [rank * inter / world, ...), the matching columns of down */
  const DgppMoeMatrixTensors* routed;   /* [n_experts * 3] gate, up, down: block FP8 (F32 or BF16 grid), NVFP4 in its three
                                           spellings, or MXFP4 */
  const DgppMoeMatrixTensors* shared;   /* [3] or null: block FP8 (slot top_k of every token), the routed experts' FP4
                                           format and width (a table entry), or MXFP8 (dense projections of its own width) */
  int64_t shared_inter;                 /* the shared expert's unsliced width (0: none) */
  const DgppTensorInfo* router_weight;  /* BF16 [n_experts, hidden], or null */
  const DgppTensorInfo* router_bias;    /* F32 or BF16 [n_experts], or null */
} DgppMoeResidentDesc;
const char* dgpp_moe_resident_last_error(void);
int dgpp_moe_resident_load(const DgppMoeResidentDesc* desc, DgppMoeResident** out);
void dgpp_moe_resident_destroy(DgppMoeResident* resident);   /* the layer and the weights */
DgppMoeLayer* dgpp_moe_resident_layer(DgppMoeResident* resident);           /* owned by the resident */
size_t dgpp_moe_resident_weight_bytes(const DgppMoeResident* resident);     /* device bytes of the weights' allocation */
int dgpp_moe_resident_inter(const DgppMoeResident* resident);               /* the rank's expert width, inter / world */

#ifdef __cplusplus
}
#endif
#endif
