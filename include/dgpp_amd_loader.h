/* Loader side of the quantized MoE path: a memory-mapped safetensors reader and the matrix views the
 * launchers consume, so that a checkpoint's bytes reach the kernels untouched (no re-encoding, no copies
 * on the host beyond the upload).
 *
 * Host code only: nothing here touches the GPU. Errors return DGPP_INVALID_ARGUMENT / DGPP_RUNTIME_ERROR
 * (dgpp_amd.h) with the message in dgpp_loader_last_error() (thread-local).
 *
 * Reference counterparts: src/loaders/safetensors.hpp (SafetensorsFile, TensorInfo),
 * src/common/dtypes.hpp:66-79 (dtype names), src/models/quant_matrix.hpp:16-96 (GlmQuantMatrix,
 * quant_scale_shifts, quant_rows_view), :117-164 (GlmFp4Matrix, fp4_rows_view). */
#ifndef DGPP_AMD_LOADER_H_
#define DGPP_AMD_LOADER_H_

#include <stddef.h>
#include <stdint.h>

#include "dgpp_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* dgpp_loader_last_error(void);

/* Element types a header may name (src/common/dtypes.hpp:66-79; "F8" and "FP8" are aliases of F8_E4M3,
 * "BOOL" of U8). Any other name fails the open. */
enum {
  DGPP_DT_F32 = 0,
  DGPP_DT_F16 = 1,
  DGPP_DT_BF16 = 2,
  DGPP_DT_F8_E4M3 = 3,
  DGPP_DT_I64 = 4,
  DGPP_DT_I32 = 5,
  DGPP_DT_U8 = 6,
  DGPP_DT_I8 = 7,
  DGPP_DT_F8_E8M0 = 8,
  DGPP_DT_U32 = 9,
  DGPP_DT_I16 = 10
};
/* Bytes of one element of `dtype`, 0 for an unknown code. */
size_t dgpp_dtype_size(int dtype);

#define DGPP_MAX_TENSOR_RANK 8

/* One tensor of an open file (src/loaders/safetensors.hpp:22-49, TensorInfo). `data` points into the
 * file's mapping and lives until the file is closed; an empty tensor's `data` is where its (empty) byte
 * range starts, possibly the end of the mapping. */
typedef struct DgppTensorInfo {
  int32_t dtype;
  int32_t rank;
  int64_t shape[DGPP_MAX_TENSOR_RANK];
  uint64_t numel;
  uint64_t nbytes;
  uint64_t file_offset; /* of the first byte, from the start of the file */
  const void* data;
} DgppTensorInfo;

typedef struct DgppSafetensors DgppSafetensors;

/* src/loaders/safetensors.hpp:103-127, :198-252: maps the file read-only and parses its header. The open
 * fails (DGPP_RUNTIME_ERROR, nothing left mapped) on a header length outside the file, malformed JSON
 * (numbers with leading zeros included), an unknown dtype, a shape or data_offsets entry that is not a
 * non-negative integer, offsets outside the payload or out of order, an element count that overflows, or
 * a byte range that is not numel * element size; more than DGPP_MAX_TENSOR_RANK dimensions likewise. */
int dgpp_safetensors_open(const char* path, DgppSafetensors** out);
/* src/loaders/safetensors.hpp:54-78 (close_mapping): unmaps; with drop_page_cache the file's pages are
 * also dropped from the page cache (advisory). Every DgppTensorInfo::data of this file dangles afterwards. */
void dgpp_safetensors_close(DgppSafetensors* f, int drop_page_cache);
int dgpp_safetensors_count(const DgppSafetensors* f);
/* Tensor names in ascending byte order of the name; NULL past the end. */
const char* dgpp_safetensors_name(const DgppSafetensors* f, int index);
/* DGPP_INVALID_ARGUMENT when the file has no tensor of that name (`out` untouched). */
int dgpp_safetensors_find(const DgppSafetensors* f, const char* name, DgppTensorInfo* out);
/* FNV-1a of the raw header JSON (src/loaders/safetensors.hpp:151-153): the shard's identity for caches. */
uint64_t dgpp_safetensors_header_fold(const DgppSafetensors* f);
/* The "__metadata__" object of the header as raw JSON text ("" when absent); lives until the close. */
const char* dgpp_safetensors_metadata_json(const DgppSafetensors* f);
/* src/loaders/safetensors.hpp:90-101: read-ahead before a one-pass copy of the tensor, and release of its
 * pages (mapping and page cache) after it. Both advisory, page-rounded. */
void dgpp_safetensors_prefetch(const DgppSafetensors* f, const DgppTensorInfo* t);
void dgpp_safetensors_discard(const DgppSafetensors* f, const DgppTensorInfo* t);

/* src/models/quant_matrix.hpp:16-52 (GlmQuantMatrix): an FP8-E4M3 matrix with an F32 block-scale grid, or
 * (scales_e8m0) the MXFP8 byte grid. Pointers may be host or device addresses: the views below only do
 * pointer arithmetic. */
typedef struct DgppQuantMatrix {
  const uint8_t* payload;     /* E4M3 [rows, cols] */
  const float* scales;        /* F32 [ceil(rows / scale_block_rows), ceil(cols / scale_block_cols)] */
  const uint8_t* scales_e8m0; /* the same grid as e8m0 bytes; exactly one of the two is set */
  int64_t rows;
  int64_t cols;
  int32_t scale_block_rows;   /* 128 in the checkpoints; 1 with scale_block_cols >= cols is the channel grid */
  int32_t scale_block_cols;
} DgppQuantMatrix;

/* src/models/quant_matrix.hpp:55-66: the grid as the launchers' log2 block sizes. Returns 1 and writes
 * rs / cs when both block sizes are powers of two and the column block is at least 16, else 0. */
int dgpp_quant_scale_shifts(const DgppQuantMatrix* m, int* rs, int* cs);
/* src/models/quant_matrix.hpp:78-96: rows [row_start, row_start + rows) as a pointer view. A start that is
 * not a multiple of the scale block's rows cannot re-anchor the grid and is rejected. */
int dgpp_quant_rows_view(const DgppQuantMatrix* m, int64_t row_start, int64_t rows, DgppQuantMatrix* out);
/* src/models/quant_matrix.hpp:144-164: K must be a positive multiple of the scale group (16 or 32); any row
 * range is a pointer view (every row carries its own scales). */
int dgpp_fp4_check_cols(int64_t cols, int scale_group);
int dgpp_fp4_rows_view(const DgppFp4Matrix* m, int64_t row_start, int64_t rows, DgppFp4Matrix* out);

/* Slices that are NOT pointer views: a copy of a HOST-resident matrix's range along rows (axis 0) or columns
 * (axis 1) into caller buffers — the tensor-parallel split of the down projection (columns), or a row split
 * that starts inside a scale block. The sliced axis of an F32 grid is re-blocked at
 * g = gcd(block, start, count): every new block lies inside one parent block and takes that block's scale
 * (src/models/quant_matrix.hpp:28-34; the reference's model loaders slice at gcd(128, I / world)), so each
 * element dequantizes to exactly the value it had in the parent. The result must still be a grid the launchers
 * take (g a power of two and at least 32, or the parent's own block), else DGPP_INVALID_ARGUMENT.
 * payload_out: count * cols (axis 0) or rows * count (axis 1) bytes; scales_out:
 * dgpp_quant_slice_scale_count floats. `out` describes the copy (its pointers are the two buffers). */
int64_t dgpp_quant_slice_scale_count(const DgppQuantMatrix* m, int axis, int64_t start, int64_t count);
int dgpp_quant_slice(const DgppQuantMatrix* m, int axis, int64_t start, int64_t count, uint8_t* payload_out,
                     float* scales_out, DgppQuantMatrix* out);
/* Column range of a HOST-resident NVFP4 / MXFP4 matrix (src/models/quant_matrix.hpp:140-150: it starts on a
 * scale-group boundary and spans whole groups). payload_out: rows * cols / 2 bytes; scales_out:
 * rows * cols / scale_group bytes. The global scale pointer is carried over. */
int dgpp_fp4_cols_slice(const DgppFp4Matrix* m, int64_t col_start, int64_t cols, uint8_t* payload_out,
                        uint8_t* scales_out, DgppFp4Matrix* out);

/* One entry of the device expert table (DgppMoeExpertView, three per expert: gate, up, down) from a
 * resident matrix. The FP8 form needs a grid dgpp_quant_scale_shifts accepts and F32 scales. */
int dgpp_expert_view_from_quant(const DgppQuantMatrix* m, DgppMoeExpertView* out);
int dgpp_expert_view_from_fp4(const DgppFp4Matrix* m, DgppMoeExpertView* out);

/* The tensors of one MoE layer of a GLM-family checkpoint under the names its exports carry
 * (src/models/glm/binding.cpp:32-54, :163-206), looked up across the given shards and checked against the
 * geometry: router `<p>mlp.gate.weight` BF16 [E, H] (and `<p>mlp.gate.e_score_correction_bias` F32 [E]); the shared
 * expert `<p>mlp.shared_experts.{gate,up,down}_proj.weight` as block FP8; routed expert e
 * `<p>mlp.experts.<e>.{gate,up,down}_proj.weight` as block FP8 (`<name>` F8_E4M3 [rows, cols] with
 * `<name>_scale_inv` F32 [ceil(rows / 128), ceil(cols / 128)]) or as NVFP4 (`<name>_packed` U8 [rows, cols / 2],
 * `<name>_scale` F8_E4M3 [rows, cols / 16], `<name>_global_scale` F32 [1]: the divisor the kernels take).
 * gate / up are [inter, hidden], down is [hidden, inter]. */
enum {
  DGPP_BIND_FP8 = 0,              /* `<name>` F8_E4M3 + `<name>_scale_inv` F32 grid */
  DGPP_BIND_NVFP4 = 1,            /* `<name>_packed`, `<name>_scale`, `<name>_global_scale` (the divisor itself) */
  DGPP_BIND_FP8_BF16_SCALES = 2,  /* as FP8 with a BF16 grid: widen it to F32 at load (exact) before the launchers see it */
  DGPP_BIND_NVFP4_MODELOPT = 3,   /* `<base>.weight` U8 [rows, cols / 2], `<base>.weight_scale` F8_E4M3 [rows, cols / 16],
                                     `<base>.weight_scale_2` F32 scalar: the kernels' divisor is 1 / weight_scale_2 */
  DGPP_BIND_MXFP8 = 4,            /* `<base>.weight` F8_E4M3, `<base>.weight_scale` U8 (e8m0) [rows, cols / 32] */
  DGPP_BIND_NVFP4_COMPRESSED = 5, /* `<base>.weight_packed` U8 [rows, cols / 2], `<base>.weight_scale` F8_E4M3 [rows, cols / 16],
                                     `<base>.weight_global_scale` F32 scalar (the divisor itself) */
  DGPP_BIND_MXFP4 = 6,            /* `<base>.weight` U8 [rows, cols / 2], `<base>.weight_scale` U8 (e8m0) [rows, cols / 32] */
  DGPP_BIND_MXFP8_SCALE_INV = 7   /* as MXFP8 with the bytes under `<base>.weight_scale_inv` */
};
typedef struct DgppMoeMatrixTensors {
  DgppTensorInfo payload;
  DgppTensorInfo scales;
  DgppTensorInfo global;   /* NVFP4 only; zeroed otherwise */
  int32_t format;          /* DGPP_BIND_* */
  int32_t file_index;      /* the shard (index into `files`) that holds the payload */
} DgppMoeMatrixTensors;
/* `p` = layer_prefix, e.g. "model.layers.3.". routed: [n_experts * 3] (gate, up, down per expert); shared: [3]
 * when shared_inter > 0 (its width; the exports use the routed experts' own); router_bias when with_bias. A missing tensor, or one whose dtype or shape differs from what
 * the geometry fixes, fails with DGPP_INVALID_ARGUMENT and a message that names it; nothing is copied: the
 * descriptions point into the shards' mappings. */
int dgpp_glm_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* layer_prefix, int n_experts,
                            int64_t hidden, int64_t inter, int routed_format, int64_t shared_inter, int with_bias,
                            DgppTensorInfo* router_weight, DgppTensorInfo* router_bias, DgppMoeMatrixTensors* shared,
                            DgppMoeMatrixTensors* routed);

/* The same for a Qwen-family MoE block (src/models/qwen/binding.cpp:26-66, :158-215); `p` = mlp_prefix, e.g.
 * "model.layers.3.mlp.": router `<p>gate.weight` BF16 [E, H]; with shared_inter > 0 the shared expert's scalar gate
 * `<p>shared_expert_gate.weight` BF16 [1, H] and `<p>shared_expert.{gate,up,down}_proj.weight` in shared_format
 * (DGPP_BIND_FP8 or DGPP_BIND_MXFP8); routed expert e `<p>experts.<e>.{gate,up,down}_proj.weight` in routed_format
 * (DGPP_BIND_FP8_BF16_SCALES, DGPP_BIND_FP8 or DGPP_BIND_NVFP4_MODELOPT; the export's `input_scale` is not looked up:
 * this path keeps BF16 activations). BF16-weight and int4 forms of these exports are not bound. */
int dgpp_qwen_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* mlp_prefix, int n_experts,
                             int64_t hidden, int64_t inter, int routed_format, int64_t shared_inter, int shared_format,
                             DgppTensorInfo* router_weight, DgppTensorInfo* shared_gate, DgppMoeMatrixTensors* shared,
                             DgppMoeMatrixTensors* routed);

/* The MXFP4 MoE block of a MiMo-family export (src/models/mimo/binding.cpp:38-42, :58-71); `p` = mlp_prefix:
 * router `<p>gate.weight` BF16 [E, H] and `<p>gate.e_score_correction_bias` F32 [E]; routed expert e
 * `<p>experts.<e>.{gate,up,down}_proj` as DGPP_BIND_MXFP4. No shared expert. */
int dgpp_mimo_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* mlp_prefix, int n_experts,
                             int64_t hidden, int64_t inter, DgppTensorInfo* router_weight, DgppTensorInfo* router_bias,
                             DgppMoeMatrixTensors* routed);
/* The MoE block of a MiniMax-family export (src/models/minimax/binding.cpp:15-35, :60-71); `p` = moe_prefix, e.g.
 * "language_model.model.layers.3.block_sparse_moe.": router `<p>gate.weight` F32 [E, H] and
 * `<p>e_score_correction_bias` F32 [E]; with shared_inter > 0 `<p>shared_experts.{gate,up,down}_proj` as
 * DGPP_BIND_MXFP8_SCALE_INV; routed expert e `<p>experts.<e>.{w1,w3,w2}` (gate, up, down in that order) as
 * DGPP_BIND_NVFP4_COMPRESSED (the export's `input_global_scale` is not looked up: this path keeps BF16 activations). */
int dgpp_minimax_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* moe_prefix, int n_experts,
                                int64_t hidden, int64_t inter, int64_t shared_inter, DgppTensorInfo* router_weight,
                                DgppTensorInfo* router_bias, DgppMoeMatrixTensors* shared, DgppMoeMatrixTensors* routed);

/* A checkpoint directory as one set of shards (src/loaders/resident_stream.hpp:257-296). With a
 * `model.safetensors.index.json` the distinct file names of its "weight_map" are the shard set (relative to the
 * directory, sub-directories included; a .safetensors file the map does not name is ignored, a named one that is
 * missing fails the open); without it every *.safetensors file of the directory itself. Shards open in ascending
 * path order; no shard at all, or a tensor name that two shards carry, fails the open (DGPP_RUNTIME_ERROR, nothing
 * left mapped). dgpp_checkpoint_shards is the array the bind functions above take; it and every DgppTensorInfo::data
 * live until the close. */
typedef struct DgppCheckpoint DgppCheckpoint;
int dgpp_checkpoint_open(const char* dir, DgppCheckpoint** out);
void dgpp_checkpoint_close(DgppCheckpoint* ck);
int dgpp_checkpoint_shard_count(const DgppCheckpoint* ck);
const DgppSafetensors* const* dgpp_checkpoint_shards(const DgppCheckpoint* ck);
const char* dgpp_checkpoint_shard_path(const DgppCheckpoint* ck, int index);
uint64_t dgpp_checkpoint_tensor_count(const DgppCheckpoint* ck);
/* DGPP_INVALID_ARGUMENT when no shard has the tensor; shard_index (nullable) receives the shard's position. */
int dgpp_checkpoint_find(const DgppCheckpoint* ck, const char* name, DgppTensorInfo* out, int* shard_index);

#ifdef __cplusplus
}
#endif

#endif /* DGPP_AMD_LOADER_H_ */
