// The C ABI (include/dgpp_amd.h): argument validation mirroring the reference launchers'
// std::invalid_argument rules, then dispatch to the kernels. Nothing here allocates or syncs.
#include <hip/hip_runtime.h>

#include <limits.h>
#include <atomic>
#include <cstdlib>
#include <mutex>
#include <string>
#include <unordered_map>

#include "../../include/dgpp_amd.h"
#include "../../include/dgpp_amd_bench.h"
#include "capi_errors.hpp"
#include "gemv_kernels.hpp"
#include "moe_misc.hpp"

using namespace dgpp_amd;

namespace {

thread_local std::string g_last_error;

int fail_arg(const std::string& what) {
  g_last_error = what;
  return DGPP_INVALID_ARGUMENT;
}
int finish(hipError_t err, const char* who) {
  if (err == hipSuccess) return DGPP_OK;
  g_last_error = std::string(who) + ": " + hipGetErrorString(err);
  (void)hipGetLastError();  // drain the sticky error like the reference's check macro
  return DGPP_RUNTIME_ERROR;
}
inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// src/kernels/fp4_gemv.cuh:110-125 (k_supported) and :771-788 (the compiled sets).
bool fp4_k_supported(int k) { return k >= 32 && k % 32 == 0 && k <= 16384; }
bool fp4_k_compiled(int k, int group) {
  static const int nv[] = {32, 64, 128, 160, 256, 320, 384, 512, 640, 768, 1024, 1536, 2048, 2560, 3072, 4096, 5120, 6144, 7168, 12288};
  static const int mx[] = {32, 64, 128, 256, 512, 576, 1024, 1152, 2048, 2304, 4096, 5120};
  if (group == 32) {
    for (int v : mx) if (v == k) return true;
    return false;
  }
  for (int v : nv) if (v == k) return true;
  return false;
}
// src/kernels/fp8_gemv.cuh:47-50: k a positive multiple of 16, 16-byte aligned payload, one row stageable.
bool fp8_shape_ok(const void* payload, int k) {
  return k > 0 && k % 16 == 0 && aligned16(payload) && stage_bytes(1, k) <= kMaxLdsBytes;
}

MatRef fp8_mat(const uint8_t* payload, const void* scales, int rs, int cs) {
  MatRef m;
  m.payload = payload;
  m.scales = scales;
  m.divisor = 1.f;
  m.rs = rs;
  m.cs = cs;
  return m;
}

}  // namespace

namespace dgpp_amd {
// The measurement switches: relaxed atomics (a harness may set one while another thread launches; every launch reads a
// switch once). A build with -DDGPP_NO_TUNE compiles them out: every switch reads 0 and dgpp_tune_set does nothing.
#ifdef DGPP_NO_TUNE
int tune_get(int) { return 0; }
#else
static std::atomic<int> g_tune[kTuneCount];
int tune_get(int key) { return key >= 0 && key < kTuneCount ? g_tune[key].load(std::memory_order_relaxed) : 0; }
#endif

hipError_t ensure_lds_impl(const void* kernel, size_t bytes) {
  static std::mutex mu;
  static std::unordered_map<const void*, size_t> raised;
  std::lock_guard<std::mutex> lock(mu);
  auto it = raised.find(kernel);
  if (it != raised.end() && it->second >= bytes) return hipSuccess;
  const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLdsBytes));
  if (err == hipSuccess) raised[kernel] = kMaxLdsBytes;
  return err;
}

hipError_t launch_dense(int fmt, const DenseArgs& a, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_dense_fmt<kFmtFp8F32>(a, s);
    case kFmtFp8E8M0: return launch_dense_fmt<kFmtFp8E8M0>(a, s);
    case kFmtNvfp4: return launch_dense_fmt<kFmtNvfp4>(a, s);
    default: return launch_dense_fmt<kFmtMxfp4>(a, s);
  }
}
hipError_t launch_dense_multi(int fmt, const DenseArgs* problems, int count, hipStream_t s) {
  return fmt == kFmtFp8E8M0 ? launch_dense_multi_fmt<kFmtFp8E8M0>(problems, count, s)
                            : launch_dense_multi_fmt<kFmtFp8F32>(problems, count, s);
}
hipError_t launch_slot_gate_up(int fmt, const SlotArgs& a, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_slot_gate_up_fmt<kFmtFp8F32>(a, s);
    case kFmtNvfp4: return launch_slot_gate_up_fmt<kFmtNvfp4>(a, s);
    default: return launch_slot_gate_up_fmt<kFmtMxfp4>(a, s);
  }
}
hipError_t launch_select_gate_up(int fmt, const SlotArgs& a, const SelectArgs& sel, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_select_gate_up_fmt<kFmtFp8F32>(a, sel, s);
    case kFmtNvfp4: return launch_select_gate_up_fmt<kFmtNvfp4>(a, sel, s);
    default: return launch_select_gate_up_fmt<kFmtMxfp4>(a, sel, s);
  }
}
hipError_t launch_slot_down(int fmt, const SlotArgs& a, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_slot_down_fmt<kFmtFp8F32>(a, s);
    case kFmtNvfp4: return launch_slot_down_fmt<kFmtNvfp4>(a, s);
    default: return launch_slot_down_fmt<kFmtMxfp4>(a, s);
  }
}
hipError_t launch_grouped(int fmt, const GroupedArgs& a, int n_segs, int z_ext, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_grouped_fmt<kFmtFp8F32>(a, n_segs, z_ext, s);
    case kFmtNvfp4: return launch_grouped_fmt<kFmtNvfp4>(a, n_segs, z_ext, s);
    default: return launch_grouped_fmt<kFmtMxfp4>(a, n_segs, z_ext, s);
  }
}
hipError_t launch_slot_chain(int fmt, const ChainArgs& c, const SelectArgs* sel, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_slot_chain_fmt<kFmtFp8F32>(c, sel, s);
    case kFmtNvfp4: return launch_slot_chain_fmt<kFmtNvfp4>(c, sel, s);
    default: return launch_slot_chain_fmt<kFmtMxfp4>(c, sel, s);
  }
}
hipError_t launch_token_down(int fmt, const TokenDownArgs& a, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_token_down_fmt<kFmtFp8F32>(a, s);
    case kFmtNvfp4: return launch_token_down_fmt<kFmtNvfp4>(a, s);
    default: return launch_token_down_fmt<kFmtMxfp4>(a, s);
  }
}
hipError_t launch_dense_mma(int fmt, const DenseArgs& a, float* ws, size_t ws_bytes, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_dense_mma_fmt<kFmtFp8F32>(a, ws, ws_bytes, s);
    case kFmtFp8E8M0: return launch_dense_mma_fmt<kFmtFp8E8M0>(a, ws, ws_bytes, s);
    case kFmtNvfp4: return launch_dense_mma_fmt<kFmtNvfp4>(a, ws, ws_bytes, s);
    default: return launch_dense_mma_fmt<kFmtMxfp4>(a, ws, ws_bytes, s);
  }
}
hipError_t launch_grouped_mma(int fmt, const GroupedArgs& a, int n_segs, int z_ext, hipStream_t s) {
  switch (fmt) {
    case kFmtFp8F32: return launch_grouped_mma_fmt<kFmtFp8F32>(a, n_segs, z_ext, s);
    case kFmtNvfp4: return launch_grouped_mma_fmt<kFmtNvfp4>(a, n_segs, z_ext, s);
    default: return launch_grouped_mma_fmt<kFmtMxfp4>(a, n_segs, z_ext, s);
  }
}
}  // namespace dgpp_amd

namespace {

// Dense projection over m rows: the vector-core GEMV (up to eight rows per pass over the weights, in chunks the LDS
// can stage; each row's chain is the same whatever the chunking) or the matrix-core form (16 rows per pass) - the
// reference's launchers move to their tensor-core forms as m grows in the same way (src/kernels/scale_gemm.cu:296-339,
// src/kernels/glm_moe_launch.hpp:363). The two forms differ in fp32 summation order, so a row's bits depend on which
// form its call takes - both are held to the same oracle tolerance. `ws` (nullable) is the split-K workspace of the
// matrix-core form.
//
// Which form, measured on this chip (cold weights; 2048 x 4096 ... 17408 x 5120, one to eight rows):
// * more rows than one vector pass holds: the matrix core (the vector core would read the weights again per pass);
// * five to eight rows: the vector core pays a dot chain per row and weight, the matrix core one decode per weight -
//   but an unsplit matrix-core launch has one block per 64 weight rows, too few to fill the chip unless the matrix is
//   large: with a split-K workspace the matrix core wins from five rows on (from three for matrices of 48 M weights and
//   more). Without one, rows of 4096 elements and more run the four parts of K side by side inside a block while the
//   row tiles fit one round of the chip (dense_mfma_team_row_groups): then six rows and more take the matrix core for
//   matrices of 8 M weights (block FP8: the vector core needs two passes there) or 32 M weights (FP4) and more, and
//   matrices of 64 M weights from four (FP8) or five (FP4) rows on; otherwise only matrices of 64 M weights and
//   more, from five rows on;
// * up to four rows (three of a large matrix): the vector core.
constexpr int kVectorPassRows = kMaxActRows;
bool dense_takes_matrix_core(int fmt, int m, int n, int k, size_t ws_bytes, bool have_ws, int from_rows) {
  if (m > kVectorPassRows || m > max_stage_rows(k)) return true;
  if (from_rows > 0 && m >= from_rows) return true;   // the caller's own boundary (the reference's mma_from_rows)
  const size_t weights = static_cast<size_t>(n) * static_cast<size_t>(k);
  int parts = 1;
  switch (fmt) {
    case kFmtFp8F32: parts = mgeom<kFmtFp8F32>(k).parts; break;
    case kFmtFp8E8M0: parts = mgeom<kFmtFp8E8M0>(k).parts; break;
    case kFmtNvfp4: parts = mgeom<kFmtNvfp4>(k).parts; break;
    default: parts = mgeom<kFmtMxfp4>(k).parts; break;
  }
  const bool split = have_ws && parts > 1 && (n + 63) / 64 < 1024 &&
                     ws_bytes >= static_cast<size_t>(parts) * m * static_cast<size_t>(n) * sizeof(float);
  if (split) return m >= 5 || (m >= 3 && weights >= (48u << 20));
  if (dense_mfma_team_row_groups(parts, m, n, true) != 0) {
    // the parts of K side by side inside a block: block FP8 from six rows on (the vector core takes two passes there),
    // FP4 from six rows on for matrices of 32 M weights and more; large matrices from four rows on
    const bool fp8 = fmt == kFmtFp8F32 || fmt == kFmtFp8E8M0;
    if (m >= 6 && weights >= ((fp8 ? 8u : 32u) << 20)) return true;
    return m >= (fp8 ? 4 : 5) && weights >= (64u << 20);
  }
  return m >= 5 && weights >= (64u << 20);
}
int dense_rows(int fmt, const uint16_t* act, size_t act_stride, const MatRef& mat, const float* global, void* out,
               size_t out_stride, int out_f32, int m, int n, int k, hipStream_t stream, const char* who, int from_rows,
               void* ws = nullptr, size_t ws_bytes = 0) {
  const int core = tune_get(kTuneCore);   // bench switch: 1 pins the vector core, 2 the matrix core
  if (core != 1 && (core == 2 || dense_takes_matrix_core(fmt, m, n, k, ws_bytes, ws != nullptr, from_rows))) {
    if ((m + kTileCols - 1) / kTileCols > 65535) return fail_arg(std::string(who) + ": grid dimension overflow");
    DenseArgs a;
    a.act = act;
    a.act_stride = act_stride;
    a.mat = mat;
    a.global = global;
    a.out = out;
    a.out_stride = out_stride;
    a.out_f32 = out_f32;
    a.m = m;
    a.n = n;
    a.k = k;
    a.once = m <= kTileCols;
    return finish(launch_dense_mma(fmt, a, static_cast<float*>(ws), ws_bytes, stream), who);
  }
  const int max_rows = max_stage_rows(k);
  const size_t esz = out_f32 ? 4 : 2;
  for (int row0 = 0; row0 < m;) {
    const int rows = std::min(max_rows, m - row0);
    DenseArgs a;
    a.act = act + static_cast<size_t>(row0) * act_stride;
    a.act_stride = act_stride;
    a.mat = mat;
    a.global = global;
    a.out = static_cast<uint8_t*>(out) + static_cast<size_t>(row0) * out_stride * esz;
    a.out_stride = out_stride;
    a.out_f32 = out_f32;
    a.m = rows;
    a.n = n;
    a.k = k;
    a.once = m <= max_rows;   // one pass over the weights
    const int rc = finish(launch_dense(fmt, a, stream), who);
    if (rc != DGPP_OK) return rc;
    row0 += rows;
  }
  return DGPP_OK;
}

int fp4_gemv(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, void* out, int out_f32, int m, int n, int k,
             void* stream) {
  // src/kernels/fp4_gemv.cu:52-67
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (!w) return fail_arg("fp4_gemv: null pointer");
  if (!act || !w->payload || !w->scales || !out) return fail_arg("fp4_gemv: null pointer");
  if (w->scale_group != 16 && w->scale_group != 32)
    return fail_arg("fp4_gemv: the scale group must be 16 (NVFP4) or 32 (MXFP4)");
  if (w->scale_group == 16 && !w->global_scale) return fail_arg("fp4_gemv: an NVFP4 matrix needs its global scale");
  if (w->rows < n || w->cols != k) return fail_arg("fp4_gemv: matrix geometry does not match n, k");
  if (!fp4_k_supported(k) || !aligned16(w->payload) || !fp4_k_compiled(k, w->scale_group))
    return fail_arg("fp4_gemv: K must be a multiple of 32 in the group's compiled set and the payload 16-byte aligned");
  MatRef mat;
  mat.payload = w->payload;
  mat.scales = w->scales;
  mat.divisor = 1.f;
  mat.rs = 0;
  mat.cs = 0;
  return dense_rows(w->scale_group == 16 ? kFmtNvfp4 : kFmtMxfp4, act, act_stride, mat, w->global_scale, out,
                    static_cast<size_t>(n), out_f32, m, n, k, as_stream(stream), "fp4_gemv", 0);
}

// src/kernels/scale_gemm.cu:280-365 (launch_scale_gemm) and :406-462 (launch_scale_gemm_grid):
// every m takes the row-independent GEMV form here.
int scale_gemm(const uint16_t* act, size_t act_stride, const uint8_t* payload, const void* scales, int e8m0, void* out,
               int out_f32, int m, int n, int k, void* stream, size_t out_stride, int rs, int cs, int last_row_only,
               int compact_row, bool grid_form, const char* who, int mma_from_rows = 0, void* ws = nullptr,
               size_t ws_bytes = 0) {
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (!act || !payload || !scales || !out) return fail_arg(std::string(who) + ": null pointer");
  if (grid_form) {
    const bool row_grid = rs == 0 && cs >= 4;
    if (!row_grid && (rs < 5 || rs > 7 || cs < 5 || cs > 7))
      return fail_arg(std::string(who) + ": rs / cs must be 5..7 (32 .. 128 blocks) or a row grid (rs = 0, cs >= 4)");
  }
  if (out_stride == 0) out_stride = static_cast<size_t>(n);
  if (out_stride < static_cast<size_t>(n)) return fail_arg(std::string(who) + ": output row stride narrower than n");
  if (compact_row < -1 || compact_row >= m || (compact_row >= 0 && last_row_only))
    return fail_arg(std::string(who) + ": invalid compact row selection");
  const size_t esz = out_f32 ? 4 : 2;
  uint8_t* o = static_cast<uint8_t*>(out);
  if (last_row_only || compact_row >= 0) {
    const int sel = compact_row >= 0 ? compact_row : m - 1;
    act += static_cast<size_t>(sel) * act_stride;
    if (last_row_only) o += static_cast<size_t>(sel) * out_stride * esz;
    m = 1;
  }
  if (grid_form && (k <= 0 || k % 16 != 0)) return fail_arg(std::string(who) + ": k must be a positive multiple of 16");
  if (k <= 0) {
    // Degenerate contraction: zero outputs (src/kernels/scale_gemm.cu:303-309).
    return finish(hipMemset2DAsync(o, out_stride * esz, 0, static_cast<size_t>(n) * esz, static_cast<size_t>(m),
                                   as_stream(stream)),
                  who);
  }
  if (!fp8_shape_ok(payload, k))
    return fail_arg(std::string(who) + ": k must be a multiple of 16 with a 16-byte aligned payload");
  const int mma_from = mma_from_rows > 0 ? mma_from_rows : 0;   // the caller's own boundary can only add matrix-core cases
  return dense_rows(e8m0 ? kFmtFp8E8M0 : kFmtFp8F32, act, act_stride, fp8_mat(payload, scales, rs, cs), nullptr, o,
                    out_stride, out_f32, m, n, k, as_stream(stream), who, mma_from, ws, ws_bytes);
}

// src/kernels/glm_moe.cu:1683-1703 (check_slot_args) and :2197-2228 (check_fp4_slot_args).
int check_slot_common(const void* x, const int32_t* ids, const DgppMoeExpertView* views, const void* out, int n_routed,
                      int k_routed, int n_shared, int k_shared, const char* who) {
  if (!x || !ids || !views || !out) return fail_arg(std::string(who) + ": null pointer");
  if (n_routed <= 0 || k_routed <= 0 || n_shared < 0 || k_shared < 0 || (n_shared > 0) != (k_shared > 0))
    return fail_arg(std::string(who) + ": degenerate dims");
  return DGPP_OK;
}
int check_fp4_slot(const void* x, const int32_t* ids, const DgppMoeExpertView* views, const void* out, int n_routed,
                   int k_routed, int n_shared, int k_shared, int shared_view_base, int fp4_group, const char* who) {
  if (fp4_group != 16 && fp4_group != 32) return fail_arg(std::string(who) + ": the fp4 scale group must be 16 or 32");
  const int rc = check_slot_common(x, ids, views, out, n_routed, k_routed, n_shared, k_shared, who);
  if (rc != DGPP_OK) return rc;
  if (!fp4_k_supported(k_routed) || !fp4_k_compiled(k_routed, fp4_group))
    return fail_arg(std::string(who) + ": routed k must be a multiple of 32 in the fp4 core's compiled set");
  if (n_shared == 0) return DGPP_OK;
  if (shared_view_base >= 0) {
    if (k_shared != k_routed) return fail_arg(std::string(who) + ": the NVFP4 shared expert's k must equal the routed k");
    return DGPP_OK;
  }
  if (k_shared % 16 != 0 || stage_bytes(1, k_shared) > kMaxLdsBytes)
    return fail_arg(std::string(who) + ": shared k must be a multiple of 16");
  return DGPP_OK;
}

SlotArgs slot_args(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                   const DgppMoeExpertView* views, void* out, int out_stride, int slots, int top_k, float limit) {
  SlotArgs a{};
  a.x = x;
  a.x_stride = x_stride;
  a.ids = ids;
  a.order = order;
  a.views = views;
  a.out = out;
  a.out_stride = out_stride;
  a.slots = slots;
  a.top_k = top_k;
  a.limit = limit;
  a.shared_view_base = -1;
  a.acc_weights = nullptr;
  a.acc_out = nullptr;
  a.once = slots <= 16 * (top_k + 1);   // a decode batch of at most 16 tokens: few slots share an expert (measured up to there)
  const int tokens = top_k >= 0 ? slots / (top_k + 1) : 0;
  a.match = order == nullptr && tokens > 1 && tokens * top_k <= 128;
  return a;
}

int grouped(int fmt, const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs, int max_rows,
            int rows_per_block, const DgppMoeExpertView* views, int which, void* out, int out_f32, size_t out_stride,
            int n, int k, void* stream, const char* who, bool mma = false, const int32_t* act_rows = nullptr,
            const float* gate_up_limit = nullptr, void* out_up = nullptr) {
  if (max_rows <= 0) return fail_arg(std::string(who) + ": max_rows must be positive");
  if (which < 0 || which > 2) return fail_arg(std::string(who) + ": which must be 0, 1 or 2");
  const unsigned z_ext = rows_per_block > 0 ? static_cast<unsigned>((max_rows + rows_per_block - 1) / rows_per_block) : 1u;
  if (n_segs > 65535 || z_ext > 65535) return fail_arg(std::string(who) + ": grid dimension overflow");
  GroupedArgs a;
  a.act = act;
  a.act_stride = act_stride;
  a.segs = segs;
  a.views = views;
  a.which = which;
  a.out = out;
  a.out_stride = out_stride;
  a.out_f32 = out_f32;
  a.n = n;
  a.k = k;
  a.rows_per_block = rows_per_block > 0 ? rows_per_block : INT_MAX;
  a.group_rows = max_stage_rows(k);
  a.act_rows = act_rows;
  a.gate_up = out_up ? 2 : (gate_up_limit != nullptr ? 1 : 0);
  a.limit = gate_up_limit ? *gate_up_limit : 0.f;
  a.out_up = out_up;
  a.once = max_rows <= (mma ? kTileCols : a.group_rows);   // every segment in one pass over its expert
  if (mma) return finish(launch_grouped_mma(fmt, a, n_segs, static_cast<int>(z_ext), as_stream(stream)), who);
  return finish(launch_grouped(fmt, a, n_segs, static_cast<int>(z_ext), as_stream(stream)), who);
}

}  // namespace

extern "C" {

const char* dgpp_last_error(void) { return g_last_error.c_str(); }
}  // extern "C"
namespace dgpp_amd {
int report_invalid(const std::string& what) { return fail_arg(what); }
int report_hip(hipError_t err, const char* who) { return finish(err, who); }
}  // namespace dgpp_amd
extern "C" {
const char* dgpp_target_arch(void) { return "gfx950"; }
int dgpp_probe_copy(void* dst, const void* src, size_t bytes, void* stream) {
  const char* who = "probe copy";
  if (bytes == 0) return DGPP_OK;
  if (!dst || !src) return fail_arg(std::string(who) + ": null pointer");
  if (bytes % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0)
    return fail_arg(std::string(who) + ": bytes and both pointers must be multiples of 16");
  return finish(run_probe_copy(dst, src, bytes, as_stream(stream)), who);
}
int dgpp_probe_read(const void* src, size_t bytes, void* sink, int nontemporal, int blocks, int span, void* stream) {
  const char* who = "probe read";
  if (bytes == 0) return DGPP_OK;
  if (!src || !sink) return fail_arg(std::string(who) + ": null pointer");
  if (bytes % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0)
    return fail_arg(std::string(who) + ": bytes and the pointer must be multiples of 16");
  return finish(run_probe_read(src, bytes, sink, nontemporal, blocks, span, as_stream(stream)), who);
}
// The switches take values only in a process that asked for them before its first call here (environment
// DGPP_AMD_BENCH=1, read once): a host that merely links the library cannot have its launches steered by another
// component's call.
int dgpp_tune_enabled(void) {
#ifndef DGPP_NO_TUNE
  static const bool on = [] {
    const char* e = std::getenv("DGPP_AMD_BENCH");
    return e != nullptr && e[0] == '1' && e[1] == '\0';
  }();
  return on ? 1 : 0;
#else
  return 0;
#endif
}
void dgpp_tune_set(int key, int value) {
#ifndef DGPP_NO_TUNE
  if (dgpp_tune_enabled() && key >= 0 && key < kTuneCount) g_tune[key].store(value, std::memory_order_relaxed);
#else
  (void)key;
  (void)value;
#endif
}
int dgpp_tune_get(int key) { return tune_get(key); }

int dgpp_moe_config_validate(const DgppMoeConfig* c) {
  // src/models/glm/moe.hpp:119-133
  if (!c) return fail_arg("GlmMoeConfig: null");
  if (c->hidden <= 0 || c->inter <= 0) return fail_arg("GlmMoeConfig: hidden/inter must be positive");
  if (c->n_experts <= 0) return fail_arg("GlmMoeConfig: n_experts must be positive");
  if (c->top_k <= 0 || c->top_k > 16) return fail_arg("GlmMoeConfig: top_k must be in [1, 16] (kernel register selection)");
  if (c->top_k > c->n_experts) return fail_arg("GlmMoeConfig: top_k must not exceed n_experts");
  if (c->n_experts > 4096) return fail_arg("GlmMoeConfig: n_experts must be <= 4096 (router smem: 2*n_experts floats)");
  if (c->n_shared_experts != 0 && c->n_shared_experts != 1) return fail_arg("GlmMoeConfig: n_shared_experts must be 0 or 1");
  if (!(c->swiglu_limit > 0)) return fail_arg("GlmMoeConfig: swiglu_limit must be positive");
  if (c->router_mode < 0 || c->router_mode > 2) return fail_arg("GlmMoeConfig: unknown router mode");
  return DGPP_OK;
}

int dgpp_launch_moe_router(const uint16_t* hidden, const uint16_t* gate, const float* bias, int32_t* ids,
                           float* weights, float* scores, float* biased, const DgppMoeConfig* cfg, int tokens,
                           void* stream, int* counters, int allow_tiled) {
  (void)counters;   // the two-launch form runs either way; the counters stay at rest, as the reference's tiled branch leaves them
  const int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (tokens <= 0) return DGPP_OK;
  const bool softmax = cfg->router_mode == DGPP_ROUTER_SOFTMAX_TOPK;
  if (!hidden || !gate || (!softmax && !bias) || !ids || !weights || !scores || !biased)
    return fail_arg("moe_router: null pointer");
  if (scores == biased) return fail_arg("moe_router: scores and biased must not alias");
  if (cfg->n_experts > 65535 || tokens > 65535) return fail_arg("moe_router: grid dimension overflow");
  int r = finish(run_router_dots(cfg->router_mode, hidden, gate, bias, scores, biased, tokens, cfg->hidden,
                                 cfg->n_experts, as_stream(stream), allow_tiled),
                 "moe_router");
  if (r != DGPP_OK) return r;
  return finish(run_router_select(cfg->router_mode, scores, biased, ids, weights, tokens, cfg->n_experts, cfg->top_k,
                                  cfg->routed_scaling_factor, cfg->norm_topk_prob ? 1 : 0, as_stream(stream)),
                "moe_router");
}

int dgpp_launch_moe_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int32_t* ids,
                                float* weights, const DgppMoeConfig* cfg, int vocab, int n_tokens, void* stream) {
  const int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (n_tokens <= 0) return DGPP_OK;
  if (!tokens || !tid2eid || !scores || !ids || !weights || vocab <= 0) return fail_arg("moe_hash_routes: null pointer");
  if (cfg->router_mode == DGPP_ROUTER_SOFTMAX_TOPK)
    return fail_arg("moe_hash_routes: the softmax router leaves logits, not scores");
  return finish(run_hash_routes(tokens, tid2eid, scores, ids, weights, n_tokens, vocab, cfg->n_experts, cfg->top_k,
                                cfg->routed_scaling_factor, cfg->norm_topk_prob ? 1 : 0, as_stream(stream)),
                "moe_hash_routes");
}

int dgpp_launch_moe_router_dots(const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                                float* biased, const DgppMoeConfig* cfg, int tokens, void* stream) {
  const int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (tokens <= 0) return DGPP_OK;
  const bool softmax = cfg->router_mode == DGPP_ROUTER_SOFTMAX_TOPK;
  if (!hidden || !gate || (!softmax && !bias) || !scores || !biased) return fail_arg("moe_router_dots: null pointer");
  if (scores == biased) return fail_arg("moe_router_dots: scores and biased must not alias");
  if (cfg->n_experts > 65535 || tokens > 65535) return fail_arg("moe_router_dots: grid dimension overflow");
  return finish(run_router_dots(cfg->router_mode, hidden, gate, bias, scores, biased, tokens, cfg->hidden, cfg->n_experts,
                                as_stream(stream)),
                "moe_router_dots");
}

int dgpp_launch_moe_router_select(const float* scores, const float* biased, int32_t* ids, float* weights,
                                  const DgppMoeConfig* cfg, int tokens, void* stream) {
  const int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (tokens <= 0) return DGPP_OK;
  if (!scores || !biased || !ids || !weights) return fail_arg("moe_router_select: null pointer");
  if (tokens > 65535) return fail_arg("moe_router_select: grid dimension overflow");
  return finish(run_router_select(cfg->router_mode, scores, biased, ids, weights, tokens, cfg->n_experts, cfg->top_k,
                                  cfg->routed_scaling_factor, cfg->norm_topk_prob ? 1 : 0, as_stream(stream)),
                "moe_router_select");
}

int dgpp_launch_moe_router_select_order(const float* scores, const float* biased, int32_t* ids, float* weights,
                                        int32_t* order, const DgppMoeConfig* cfg, int tokens, int shared_early,
                                        void* stream) {
  const char* who = "moe_router_select_order";
  const int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (tokens <= 0) return DGPP_OK;
  if (!scores || !biased || !ids || !weights) return fail_arg(std::string(who) + ": null pointer");
  const int slots = tokens * (cfg->top_k + 1);
  if (order != nullptr && slots > 1024) return fail_arg(std::string(who) + ": at most 1024 slots");
  if (order != nullptr && tokens <= 16 && cfg->n_experts <= 8 * 64)
    return finish(run_router_select_order(cfg->router_mode, scores, biased, ids, weights, order, tokens, cfg->n_experts,
                                          cfg->top_k, cfg->routed_scaling_factor, cfg->norm_topk_prob ? 1 : 0,
                                          shared_early, as_stream(stream)),
                  who);
  const int rc2 = dgpp_launch_moe_router_select(scores, biased, ids, weights, cfg, tokens, stream);
  if (rc2 != DGPP_OK || order == nullptr) return rc2;
  return finish(run_slot_order(ids, order, nullptr, slots, cfg->top_k, cfg->n_experts, shared_early, as_stream(stream)),
                who);
}

int dgpp_launch_moe_swiglu_clamp(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, float limit,
                                 void* stream) {
  if (n <= 0) return DGPP_OK;
  if (!gate || !up || !out) return fail_arg("moe_swiglu: null pointer");
  return finish(run_swiglu_clamp(gate, up, out, n, limit, as_stream(stream)), "moe_swiglu");
}

int dgpp_launch_moe_gather_rows(const uint16_t* src, const int32_t* rows, uint16_t* dst, int n_rows, int hidden,
                                void* stream) {
  if (n_rows <= 0) return DGPP_OK;
  if (!src || !rows || !dst) return fail_arg("moe_gather: null pointer");
  return finish(run_gather_rows(src, rows, dst, n_rows, hidden, as_stream(stream)), "moe_gather");
}

int dgpp_launch_moe_accum(float* acc, const float* y, const int32_t* rows, const float* row_weights, int n_rows,
                          int hidden, void* stream) {
  if (n_rows <= 0) return DGPP_OK;
  if (!acc || !y || !rows || !row_weights) return fail_arg("moe_accum: null pointer");
  return finish(run_accum(acc, y, rows, row_weights, n_rows, hidden, as_stream(stream)), "moe_accum");
}

int dgpp_launch_moe_round_bf16(uint16_t* out, const float* acc, int64_t n, void* stream) {
  if (n <= 0) return DGPP_OK;
  if (!out || !acc) return fail_arg("moe_round: null pointer");
  return finish(run_round_bf16(out, acc, n, as_stream(stream)), "moe_round");
}

int dgpp_launch_moe_segment(const int32_t* ids, int tokens, int top_k, int n_experts, int32_t* rows,
                            int32_t* slot_row, DgppMoeSegment* segs, void* stream) {
  if (tokens <= 0) return DGPP_OK;
  if (!ids || !rows || !slot_row || !segs) return fail_arg("moe segment: null pointer");
  if (top_k < 1 || top_k > 16 || n_experts < 1 || n_experts > 1024)
    return fail_arg("moe segment: top_k or n_experts out of range");
  return finish(run_segment(ids, tokens, top_k, n_experts, rows, slot_row, segs, as_stream(stream)), "moe segment");
}

int dgpp_moe_tile_list_capacity(int n_segs, int total_rows, int tile_rows) {
  return n_segs + (total_rows + tile_rows - 1) / tile_rows;
}

int dgpp_launch_moe_tile_list(const DgppMoeSegment* segs, int n_segs, int tile_rows, DgppMoeTile* tiles,
                              int32_t* count, void* stream) {
  if (!segs || !tiles || !count) return fail_arg("moe tile list: null pointer");
  if (n_segs < 1 || n_segs > 65535 || tile_rows < 1) return fail_arg("moe tile list: n_segs or tile_rows out of range");
  return finish(run_tile_list(segs, n_segs, tile_rows, tiles, count, as_stream(stream)), "moe tile list");
}

int dgpp_moe_run_groups_max(int slots) { return slots / 17 + 1; }

int dgpp_launch_moe_slot_order(const int32_t* ids, int32_t* order, int slots, int top_k, int n_experts, void* stream,
                               int shared_early, int32_t* runs) {
  if (slots <= 0) return DGPP_OK;
  if (!ids || !order) return fail_arg("moe_slot_order: null");
  if (slots > 1024) return fail_arg("moe_slot_order: more slots than one block");
  return finish(run_slot_order(ids, order, runs, slots, top_k, n_experts, shared_early ? 1 : 0, as_stream(stream)),
                "moe_slot_order");
}

int dgpp_minimax_router(const uint16_t* x, const float* gate, const float* bias, int rows, int hidden, int experts, int topk,
                        float factor, float* scores, int32_t* ids, float* weights, void* stream) {
  const char* who = "minimax_router";
  if (rows <= 0) return DGPP_OK;
  if (experts <= 0 || topk <= 0 || topk > 16 || topk > experts) return fail_arg(std::string(who) + ": MiniMax router shape");
  if (experts > 4096) return fail_arg(std::string(who) + ": at most 4096 experts (the score row lives in a wavefront's registers)");
  if (hidden <= 0 || rows > 65535) return fail_arg(std::string(who) + ": degenerate dims");
  if (!x || !gate || !bias || !scores || !ids || !weights) return fail_arg(std::string(who) + ": null pointer");
  return finish(run_minimax_router(x, gate, bias, rows, hidden, experts, topk, factor, scores, ids, weights, as_stream(stream)), who);
}
int dgpp_minimax_compact_segments(const DgppMoeSegment* input, DgppMoeSegment* output, int experts, int capacity,
                                  void* stream) {
  if (!input || !output || input == output || experts < 1 || experts > 1024 || capacity < 1 || capacity > experts)
    return fail_arg("MiniMax segment compaction geometry");
  return finish(run_compact_segments(input, output, experts, capacity, as_stream(stream)), "minimax_compact_segments");
}

static int accum_ordered(void* out, int out_f32, const void* down, size_t down_stride, const int32_t* slot_row,
                         const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens, int top_k,
                         int hidden, void* stream, int down_bf16 = 0) {
  if (tokens <= 0) return DGPP_OK;
  if (!out || !down || !slot_row || !slot_ids || !slot_w) return fail_arg("moe accum ordered: null pointer");
  if (top_k < 1 || top_k > 16) return fail_arg("moe accum ordered: top_k outside [1, 16]");
  return finish(run_accum_ordered(out, out_f32, down, down_bf16, down_stride, slot_row, slot_ids, slot_w, shared_row0, tokens,
                                  top_k, hidden, as_stream(stream)),
                "moe accum ordered");
}
int dgpp_launch_moe_accum_ordered_bf16down(uint16_t* out, const uint16_t* down, size_t down_stride, const int32_t* slot_row,
                                           const int32_t* slot_ids, const float* slot_w, int tokens, int top_k, int hidden,
                                           void* stream) {
  return accum_ordered(out, 0, down, down_stride, slot_row, slot_ids, slot_w, -1, tokens, top_k, hidden, stream, 1);
}
int dgpp_launch_moe_accum_ordered_f32_bf16down(float* out, const uint16_t* down, size_t down_stride, const int32_t* slot_row,
                                               const int32_t* slot_ids, const float* slot_w, int tokens, int top_k, int hidden,
                                               void* stream) {
  return accum_ordered(out, 1, down, down_stride, slot_row, slot_ids, slot_w, -1, tokens, top_k, hidden, stream, 1);
}
int dgpp_launch_moe_accum_ordered(uint16_t* out, const float* down, size_t down_stride, const int32_t* slot_row,
                                  const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                                  int top_k, int hidden, void* stream) {
  return accum_ordered(out, 0, down, down_stride, slot_row, slot_ids, slot_w, shared_row0, tokens, top_k, hidden, stream);
}
int dgpp_launch_moe_accum_ordered_f32(float* out, const float* down, size_t down_stride, const int32_t* slot_row,
                                      const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                                      int top_k, int hidden, void* stream) {
  return accum_ordered(out, 1, down, down_stride, slot_row, slot_ids, slot_w, shared_row0, tokens, top_k, hidden, stream);
}

int dgpp_launch_moe_slot_accum(uint16_t* out, const float* contrib, const float* weights, int tokens, int hidden,
                               int top_k, void* stream) {
  if (tokens <= 0) return DGPP_OK;
  if (!out || !contrib || !weights) return fail_arg("moe_slot_accum: null pointer");
  return finish(run_slot_accum(out, 0, 1, contrib, weights, tokens, hidden, top_k, as_stream(stream)), "moe_slot_accum");
}
int dgpp_launch_moe_slot_accum_routed_f32(float* out, const float* contrib, const float* weights, int tokens,
                                          int hidden, int top_k, void* stream) {
  if (tokens <= 0) return DGPP_OK;
  if (!out || !contrib || !weights) return fail_arg("moe_slot_accum_routed_f32: null pointer");
  return finish(run_slot_accum(out, 1, 0, contrib, weights, tokens, hidden, top_k, as_stream(stream)),
                "moe_slot_accum_routed_f32");
}

int dgpp_launch_moe_slot_accum_routed_bf16(uint16_t* out, const float* contrib, const float* weights, int tokens,
                                           int hidden, int top_k, void* stream) {
  if (tokens <= 0) return DGPP_OK;
  if (!out || !contrib || !weights) return fail_arg("moe_slot_accum_routed_bf16: null pointer");
  return finish(run_slot_accum(out, 0, 0, contrib, weights, tokens, hidden, top_k, as_stream(stream)),
                "moe_slot_accum_routed_bf16");
}

namespace {
// The pass selector of the *_ex decode-slot launchers: bit 0 the routed slots, bit 1 the shared slots.
// A request that cannot be carried out is an error, never dropped: a pass selector outside 1..3, a shared pass
// without a shared expert, an accumulation target without the shared pass that would write it.
int check_passes(int passes, int n_shared, const float* acc_w, const uint16_t* acc_o, const char* who) {
  if (passes < 1 || passes > 3) return fail_arg(std::string(who) + ": passes must be 1 (routed), 2 (shared) or 3 (both)");
  if (passes == 2 && n_shared == 0) return fail_arg(std::string(who) + ": the shared pass was asked for and there is no shared expert");
  if ((acc_w == nullptr) != (acc_o == nullptr))
    return fail_arg(std::string(who) + ": the accumulation needs both its weights and its output row");
  if (acc_o != nullptr && (n_shared == 0 || !(passes & 2)))
    return fail_arg(std::string(who) + ": the accumulation rides the shared pass, which this call does not run");
  return DGPP_OK;
}
}  // namespace

int dgpp_launch_moe_slot_gate_up_swiglu(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                        const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                        int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                        const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                        int act_stride, int slots, int top_k, float limit, void* stream, int sh_rs,
                                        int sh_cs) {
  return dgpp_launch_moe_slot_gate_up_swiglu_ex(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                                sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act, act_stride,
                                                slots, top_k, limit, stream, sh_rs, sh_cs, 3);
}

int dgpp_launch_moe_slot_gate_up_swiglu_ex(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                           const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                           int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                           const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                           int act_stride, int slots, int top_k, float limit, void* stream, int sh_rs,
                                           int sh_cs, int passes) {
  const char* who = "moe_slot_gate_up";
  if (slots <= 0) return DGPP_OK;
  int rc = check_passes(passes, n_shared, nullptr, nullptr, who);
  if (rc != DGPP_OK) return rc;
  rc = check_slot_common(x, ids, views, act, n_routed, k_routed, n_shared, k_shared, who);
  if (rc != DGPP_OK) return rc;
  if (k_routed % 16 != 0 || stage_bytes(1, k_routed) > kMaxLdsBytes)
    return fail_arg(std::string(who) + ": k must be a multiple of 16 (16B-aligned payloads)");
  if (n_shared > 0 && (!sh_gate_payload || !sh_gate_scales || !sh_up_payload || !sh_up_scales ||
                       !fp8_shape_ok(sh_gate_payload, k_shared) || !fp8_shape_ok(sh_up_payload, k_shared)))
    return fail_arg(std::string(who) + ": shared payloads must be 16B-aligned with k % 16 == 0");
  if (act_stride < n_routed || act_stride < n_shared) return fail_arg(std::string(who) + ": act_stride below n");
  SlotArgs a = slot_args(x, x_stride, ids, order, views, act, act_stride, slots, top_k, limit);
  a.n = n_routed;
  a.k = k_routed;
  a.want_shared = 0;
  rc = (passes & 1) ? finish(launch_slot_gate_up(kFmtFp8F32, a, as_stream(stream)), who) : DGPP_OK;
  if (rc != DGPP_OK || n_shared == 0 || !(passes & 2)) return rc;
  a.n = n_shared;
  a.k = k_shared;
  a.want_shared = 1;
  a.sh[0] = fp8_mat(sh_gate_payload, sh_gate_scales, sh_rs, sh_cs);
  a.sh[1] = fp8_mat(sh_up_payload, sh_up_scales, sh_rs, sh_cs);
  return finish(launch_slot_gate_up(kFmtFp8F32, a, as_stream(stream)), who);
}

namespace {
// The limits of select_gate_up_kernel: one token, its score row fits a wavefront's registers, and the
// decode form of the gate/up kernel (fast set-up) applies.
bool select_gate_up_fits(const SlotArgs& a, int tokens, int n_experts) {
  return tokens == 1 && a.top_k <= kWave && n_experts <= 8 * kWave && tune_get(kTuneCore) != 2 &&
         tune_get(kTuneSplitStage) != 1 && tune_get(kTuneSelectAlone) != 1 && a.k <= 8 * kSplitStageVecs * kBlockThreads &&
         (a.x_stride & 7u) == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0;
}

int select_gate_up(int fmt, const float* scores, const float* biased, int32_t* ids, float* weights, const DgppMoeConfig* cfg,
                   int tokens, const uint16_t* x, size_t x_stride, const DgppMoeExpertView* views, int n_routed,
                   int k_routed, uint16_t* act, int act_stride, float limit, void* stream, int fp4_group, const char* who) {
  int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (tokens <= 0) return DGPP_OK;
  if (!scores || !biased || !ids || !weights) return fail_arg(std::string(who) + ": null pointer");
  if (tokens > 65535) return fail_arg(std::string(who) + ": grid dimension overflow");
  const int slots = tokens * (cfg->top_k + 1);
  SlotArgs a = slot_args(x, x_stride, ids, nullptr, views, act, act_stride, slots, cfg->top_k, limit);
  a.n = n_routed;
  a.k = k_routed;
  a.want_shared = 0;
  if (!x || !views || !act || n_routed <= 0 || k_routed <= 0 || act_stride < n_routed || !select_gate_up_fits(a, tokens, cfg->n_experts)) {
    // outside the one-launch form (or invalid: the two launchers say why)
    rc = dgpp_launch_moe_router_select(scores, biased, ids, weights, cfg, tokens, stream);
    if (rc != DGPP_OK) return rc;
    if (fmt == kFmtFp8F32)
      return dgpp_launch_moe_slot_gate_up_swiglu(x, x_stride, ids, nullptr, views, n_routed, k_routed, 0, 0, nullptr, nullptr,
                                                 nullptr, nullptr, act, act_stride, slots, cfg->top_k, limit, stream, 7, 7);
    return dgpp_launch_moe_slot_gate_up_swiglu_fp4(x, x_stride, ids, nullptr, views, n_routed, k_routed, 0, 0, nullptr, nullptr,
                                                   nullptr, nullptr, act, act_stride, slots, cfg->top_k, limit, stream, -1,
                                                   fp4_group, 7, 7);
  }
  if (fmt == kFmtFp8F32) {
    rc = check_slot_common(x, ids, views, act, n_routed, k_routed, 0, 0, who);
    if (rc != DGPP_OK) return rc;
    if (k_routed % 16 != 0 || stage_bytes(1, k_routed) > kMaxLdsBytes)
      return fail_arg(std::string(who) + ": k must be a multiple of 16 (16B-aligned payloads)");
  } else {
    rc = check_fp4_slot(x, ids, views, act, n_routed, k_routed, 0, 0, -1, fp4_group, who);
    if (rc != DGPP_OK) return rc;
  }
  SelectArgs sel;
  sel.scores = scores;
  sel.biased = biased;
  sel.ids = ids;
  sel.weights = weights;
  sel.mode = cfg->router_mode;
  sel.n_experts = cfg->n_experts;
  sel.scaling = cfg->routed_scaling_factor;
  sel.norm_topk = cfg->norm_topk_prob ? 1 : 0;
  return finish(launch_select_gate_up(fmt, a, sel, as_stream(stream)), who);
}
}  // namespace

int dgpp_launch_moe_select_gate_up_swiglu(const float* scores, const float* biased, int32_t* ids, float* weights,
                                          const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                          const DgppMoeExpertView* views, int n_routed, int k_routed, uint16_t* act,
                                          int act_stride, float limit, void* stream) {
  return select_gate_up(kFmtFp8F32, scores, biased, ids, weights, cfg, tokens, x, x_stride, views, n_routed, k_routed, act,
                        act_stride, limit, stream, 0, "moe_select_gate_up");
}
int dgpp_launch_moe_select_gate_up_swiglu_fp4(const float* scores, const float* biased, int32_t* ids, float* weights,
                                              const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                              const DgppMoeExpertView* views, int n_routed, int k_routed, uint16_t* act,
                                              int act_stride, float limit, void* stream, int fp4_group) {
  if (fp4_group != 16 && fp4_group != 32) return fail_arg("moe_select_gate_up_fp4: fp4_group must be 16 or 32");
  return select_gate_up(fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4, scores, biased, ids, weights, cfg, tokens, x, x_stride, views,
                        n_routed, k_routed, act, act_stride, limit, stream, fp4_group, "moe_select_gate_up_fp4");
}

int dgpp_launch_moe_slot_down(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                              const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared, int k_shared,
                              const uint8_t* sh_payload, const float* sh_scales, float* out, int out_stride, int slots,
                              int top_k, void* stream, int sh_rs, int sh_cs) {
  return dgpp_launch_moe_slot_down_ex(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared, sh_payload,
                                      sh_scales, out, out_stride, slots, top_k, stream, sh_rs, sh_cs, 3, nullptr, nullptr);
}

int dgpp_launch_moe_slot_down_ex(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                 const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared, int k_shared,
                                 const uint8_t* sh_payload, const float* sh_scales, float* out, int out_stride, int slots,
                                 int top_k, void* stream, int sh_rs, int sh_cs, int passes, const float* acc_w,
                                 uint16_t* acc_o) {
  const char* who = "moe_slot_down";
  if (slots <= 0) return DGPP_OK;
  int rc = check_passes(passes, n_shared, acc_w, acc_o, who);
  if (rc != DGPP_OK) return rc;
  rc = check_slot_common(act, ids, views, out, n_routed, k_routed, n_shared, k_shared, who);
  if (rc != DGPP_OK) return rc;
  if (k_routed % 16 != 0 || stage_bytes(1, k_routed) > kMaxLdsBytes)
    return fail_arg(std::string(who) + ": k must be a multiple of 16 (16B-aligned payloads)");
  if (n_shared > 0 && (!sh_payload || !sh_scales || !fp8_shape_ok(sh_payload, k_shared)))
    return fail_arg(std::string(who) + ": shared payload must be 16B-aligned with k % 16 == 0");
  if (out_stride < n_routed || out_stride < n_shared) return fail_arg(std::string(who) + ": out_stride below n");
  SlotArgs a = slot_args(act, act_stride, ids, order, views, out, out_stride, slots, top_k, 0.f);
  a.n = n_routed;
  a.k = k_routed;
  a.want_shared = 0;
  rc = (passes & 1) ? finish(launch_slot_down(kFmtFp8F32, a, as_stream(stream)), who) : DGPP_OK;
  if (rc != DGPP_OK || n_shared == 0 || !(passes & 2)) return rc;
  a.n = n_shared;
  a.k = k_shared;
  a.want_shared = 1;
  if (acc_w && acc_o) a.acc_weights = acc_w, a.acc_out = acc_o;
  a.sh[0] = fp8_mat(sh_payload, sh_scales, sh_rs, sh_cs);
  return finish(launch_slot_down(kFmtFp8F32, a, as_stream(stream)), who);
}

int dgpp_launch_moe_slot_gate_up_swiglu_fp4(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                            const int32_t* order, const DgppMoeExpertView* views, int n_routed,
                                            int k_routed, int n_shared, int k_shared, const uint8_t* sh_gate_payload,
                                            const float* sh_gate_scales, const uint8_t* sh_up_payload,
                                            const float* sh_up_scales, uint16_t* act, int act_stride, int slots,
                                            int top_k, float limit, void* stream, int shared_view_base, int fp4_group,
                                            int sh_rs, int sh_cs) {
  return dgpp_launch_moe_slot_gate_up_swiglu_fp4_ex(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                                    sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act,
                                                    act_stride, slots, top_k, limit, stream, shared_view_base, fp4_group,
                                                    sh_rs, sh_cs, 3);
}

int dgpp_launch_moe_slot_gate_up_swiglu_fp4_ex(const uint16_t* x, size_t x_stride, const int32_t* ids,
                                               const int32_t* order, const DgppMoeExpertView* views, int n_routed,
                                               int k_routed, int n_shared, int k_shared, const uint8_t* sh_gate_payload,
                                               const float* sh_gate_scales, const uint8_t* sh_up_payload,
                                               const float* sh_up_scales, uint16_t* act, int act_stride, int slots,
                                               int top_k, float limit, void* stream, int shared_view_base, int fp4_group,
                                               int sh_rs, int sh_cs, int passes) {
  const char* who = "moe_slot_gate_up_fp4";
  if (slots <= 0) return DGPP_OK;
  int rc = check_passes(passes, n_shared, nullptr, nullptr, who);
  if (rc != DGPP_OK) return rc;
  rc = check_fp4_slot(x, ids, views, act, n_routed, k_routed, n_shared, k_shared, shared_view_base, fp4_group, who);
  if (rc != DGPP_OK) return rc;
  const bool shared_fp4 = shared_view_base >= 0;
  if (n_shared > 0 && !shared_fp4 &&
      (!sh_gate_payload || !sh_gate_scales || !sh_up_payload || !sh_up_scales ||
       !fp8_shape_ok(sh_gate_payload, k_shared) || !fp8_shape_ok(sh_up_payload, k_shared)))
    return fail_arg(std::string(who) + ": shared payloads must be 16B-aligned with k % 16 == 0");
  if (act_stride < n_routed || act_stride < n_shared) return fail_arg(std::string(who) + ": act_stride below n");
  const int fmt = fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4;
  SlotArgs a = slot_args(x, x_stride, ids, order, views, act, act_stride, slots, top_k, limit);
  a.n = n_routed;
  a.k = k_routed;
  a.want_shared = 0;
  rc = (passes & 1) ? finish(launch_slot_gate_up(fmt, a, as_stream(stream)), who) : DGPP_OK;
  if (rc != DGPP_OK || n_shared == 0 || !(passes & 2)) return rc;
  a.n = n_shared;
  a.k = k_shared;
  a.want_shared = 1;
  if (shared_fp4) {
    a.shared_view_base = shared_view_base;
    return finish(launch_slot_gate_up(fmt, a, as_stream(stream)), who);
  }
  a.sh[0] = fp8_mat(sh_gate_payload, sh_gate_scales, sh_rs, sh_cs);
  a.sh[1] = fp8_mat(sh_up_payload, sh_up_scales, sh_rs, sh_cs);
  return finish(launch_slot_gate_up(kFmtFp8F32, a, as_stream(stream)), who);
}

int dgpp_launch_moe_slot_gate_up_swiglu_mixed(const uint16_t* x, size_t x_stride, const int32_t* ids, const int32_t* order,
                                              const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                              int k_shared, const uint8_t* sh_gate_payload, const float* sh_gate_scales,
                                              const uint8_t* sh_up_payload, const float* sh_up_scales, uint16_t* act,
                                              int act_stride, int slots, int top_k, float limit, int gate_fp4, int fp4_group,
                                              void* stream, int sh_rs, int sh_cs) {
  const char* who = "moe_slot_gate_up_mixed";
  if (slots <= 0) return DGPP_OK;
  if (fp4_group != 16)
    return fail_arg(std::string(who) + ": the per-projection form mixes fp8 with NVFP4 (group 16)");
  int rc = check_fp4_slot(x, ids, views, act, n_routed, k_routed, n_shared, k_shared, -1, fp4_group, who);
  if (rc != DGPP_OK) return rc;
  if (k_routed % 16 != 0) return fail_arg(std::string(who) + ": k must be a multiple of 16 (the fp8 core)");
  if (n_shared > 0 && (!sh_gate_payload || !sh_gate_scales || !sh_up_payload || !sh_up_scales ||
                       !fp8_shape_ok(sh_gate_payload, k_shared) || !fp8_shape_ok(sh_up_payload, k_shared)))
    return fail_arg(std::string(who) + ": shared payloads must be 16B-aligned with k % 16 == 0");
  if (act_stride < n_routed || act_stride < n_shared) return fail_arg(std::string(who) + ": act_stride below n");
  if (stage_bytes(2, k_routed) + 4096 > kMaxLdsBytes) return fail_arg(std::string(who) + ": k beyond what the two stages hold");
  SlotArgs a = slot_args(x, x_stride, ids, order, views, act, act_stride, slots, top_k, limit);
  a.n = n_routed;
  a.k = k_routed;
  a.want_shared = 0;
  a.match = 0;   // one slot per block
  rc = finish(launch_slot_gate_up_mixed(a, gate_fp4, as_stream(stream)), who);
  if (rc != DGPP_OK || n_shared == 0) return rc;
  a = slot_args(x, x_stride, ids, order, views, act, act_stride, slots, top_k, limit);
  a.n = n_shared;   // the shared slots run the fp8 core on both projections, as the fp4 launcher's do
  a.k = k_shared;
  a.want_shared = 1;
  a.sh[0] = fp8_mat(sh_gate_payload, sh_gate_scales, sh_rs, sh_cs);
  a.sh[1] = fp8_mat(sh_up_payload, sh_up_scales, sh_rs, sh_cs);
  return finish(launch_slot_gate_up(kFmtFp8F32, a, as_stream(stream)), who);
}

int dgpp_launch_moe_slot_down_fp4(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                  const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                  int k_shared, const uint8_t* sh_payload, const float* sh_scales, float* out,
                                  int out_stride, int slots, int top_k, void* stream, int shared_view_base,
                                  int fp4_group, int sh_rs, int sh_cs, int* tile_counter) {
  return dgpp_launch_moe_slot_down_fp4_ex(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                          sh_payload, sh_scales, out, out_stride, slots, top_k, stream, shared_view_base,
                                          fp4_group, sh_rs, sh_cs, tile_counter, 3, nullptr, nullptr);
}

int dgpp_launch_moe_slot_down_fp4_ex(const uint16_t* act, size_t act_stride, const int32_t* ids, const int32_t* order,
                                     const DgppMoeExpertView* views, int n_routed, int k_routed, int n_shared,
                                     int k_shared, const uint8_t* sh_payload, const float* sh_scales, float* out,
                                     int out_stride, int slots, int top_k, void* stream, int shared_view_base,
                                     int fp4_group, int sh_rs, int sh_cs, int* tile_counter, int passes,
                                     const float* acc_w, uint16_t* acc_o) {
  const char* who = "moe_slot_down_fp4";
  if (slots <= 0) return DGPP_OK;
  if (tile_counter == nullptr) return fail_arg(std::string(who) + ": the stealing counter pair is required");
  int rc = check_passes(passes, n_shared, acc_w, acc_o, who);
  if (rc != DGPP_OK) return rc;
  rc = check_fp4_slot(act, ids, views, out, n_routed, k_routed, n_shared, k_shared, shared_view_base, fp4_group, who);
  if (rc != DGPP_OK) return rc;
  const bool shared_fp4 = shared_view_base >= 0;
  if (n_shared > 0 && !shared_fp4 && (!sh_payload || !sh_scales || !fp8_shape_ok(sh_payload, k_shared)))
    return fail_arg(std::string(who) + ": shared payload must be 16B-aligned with k % 16 == 0");
  if (out_stride < n_routed || out_stride < n_shared) return fail_arg(std::string(who) + ": out_stride below n");
  const int fmt = fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4;
  SlotArgs a = slot_args(act, act_stride, ids, order, views, out, out_stride, slots, top_k, 0.f);
  a.n = n_routed;
  a.k = k_routed;
  a.want_shared = 0;
  rc = (passes & 1) ? finish(launch_slot_down(fmt, a, as_stream(stream)), who) : DGPP_OK;
  if (rc != DGPP_OK || n_shared == 0 || !(passes & 2)) return rc;
  a.n = n_shared;
  a.k = k_shared;
  a.want_shared = 1;
  if (acc_w && acc_o) a.acc_weights = acc_w, a.acc_out = acc_o;
  if (shared_fp4) {
    a.shared_view_base = shared_view_base;
    return finish(launch_slot_down(fmt, a, as_stream(stream)), who);
  }
  a.sh[0] = fp8_mat(sh_payload, sh_scales, sh_rs, sh_cs);
  return finish(launch_slot_down(kFmtFp8F32, a, as_stream(stream)), who);
}

// Routed down + ordered accumulation in one launch (no counterpart in the reference, which runs
// launch_moe_slot_down* and launch_moe_slot_accum_routed_* back to back).
static int slot_down_accum(int fmt, const uint16_t* act, size_t act_stride, const int32_t* ids,
                           const DgppMoeExpertView* views, int n, int k, int tokens, int top_k, const float* weights,
                           uint16_t* out_bf16, float* out_f32, void* stream, const char* who) {
  if (tokens <= 0) return DGPP_OK;
  if (!act || !ids || !views || !weights || (!out_bf16 && !out_f32)) return fail_arg(std::string(who) + ": null pointer");
  if (n <= 0 || k <= 0 || top_k <= 0 || top_k > 16) return fail_arg(std::string(who) + ": degenerate dims (top_k 1..16)");
  if (tokens > 65535) return fail_arg(std::string(who) + ": grid dimension overflow");
  if (act_stride < static_cast<size_t>(k)) return fail_arg(std::string(who) + ": act_stride below k");
  if (static_cast<size_t>(top_k) * (stage_bytes(1, k) + 8 * 64 * sizeof(float)) > kMaxLdsBytes)
    return fail_arg(std::string(who) + ": top_k activation rows of k elements exceed the LDS budget");
  TokenDownArgs a;
  a.act = act;
  a.act_stride = act_stride;
  a.ids = ids;
  a.views = views;
  a.weights = weights;
  a.out = out_f32 ? static_cast<void*>(out_f32) : static_cast<void*>(out_bf16);
  a.out_f32 = out_f32 != nullptr;
  a.n = n;
  a.k = k;
  a.tokens = tokens;
  a.top_k = top_k;
  return finish(launch_token_down(fmt, a, as_stream(stream)), who);
}
int dgpp_launch_moe_slot_down_accum(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                    const DgppMoeExpertView* views, int n, int k, int tokens, int top_k,
                                    const float* weights, uint16_t* out_bf16, float* out_f32, void* stream) {
  const char* who = "moe_slot_down_accum";
  if (tokens > 0 && (k % 16 != 0 || stage_bytes(1, k) > kMaxLdsBytes))
    return fail_arg(std::string(who) + ": k must be a multiple of 16 (16B-aligned payloads)");
  return slot_down_accum(kFmtFp8F32, act, act_stride, ids, views, n, k, tokens, top_k, weights, out_bf16, out_f32, stream, who);
}
int dgpp_launch_moe_slot_down_accum_fp4(const uint16_t* act, size_t act_stride, const int32_t* ids,
                                        const DgppMoeExpertView* views, int n, int k, int tokens, int top_k,
                                        const float* weights, uint16_t* out_bf16, float* out_f32, void* stream,
                                        int fp4_group) {
  const char* who = "moe_slot_down_accum_fp4";
  if (fp4_group != 16 && fp4_group != 32) return fail_arg(std::string(who) + ": the fp4 scale group must be 16 or 32");
  if (tokens > 0 && (!fp4_k_supported(k) || !fp4_k_compiled(k, fp4_group)))
    return fail_arg(std::string(who) + ": k must be a multiple of 32 in the fp4 core's compiled set");
  return slot_down_accum(fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4, act, act_stride, ids, views, n, k, tokens, top_k, weights,
                         out_bf16, out_f32, stream, who);
}

// The routed chain of a small decode batch in one launch (no counterpart in the reference, which runs
// launch_moe_slot_gate_up_swiglu*, launch_moe_slot_down* and launch_moe_slot_accum_routed_* back to back). Problems
// outside the one-launch form run as the two launches it stands for; the bits are the same either way.
static int slot_chain(int fmt, const uint16_t* x, size_t x_stride, const int32_t* ids, const DgppMoeExpertView* views,
                      int inter, int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                      const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status, unsigned spins,
                      void* stream, int fp4_group, const char* who, const SelectArgs* sel = nullptr,
                      const DgppMoeConfig* cfg = nullptr) {
  if (tokens <= 0) return DGPP_OK;
  if (!x || !ids || !views || !act || !weights || (!out_bf16 && !out_f32)) return fail_arg(std::string(who) + ": null pointer");
  if (inter <= 0 || hidden <= 0 || top_k <= 0 || top_k > 16) return fail_arg(std::string(who) + ": degenerate dims (top_k 1..16)");
  if (act_stride < inter) return fail_arg(std::string(who) + ": act_stride below the expert width");
  ChainArgs c{};
  const int slots = tokens * (top_k + 1);
  c.gu = slot_args(x, x_stride, ids, nullptr, views, act, act_stride, slots, top_k, limit);
  c.gu.n = inter;
  c.gu.k = hidden;
  c.dn.act = act;
  c.dn.act_stride = static_cast<size_t>(act_stride);
  c.dn.ids = ids;
  c.dn.views = views;
  c.dn.weights = weights;
  c.dn.out = out_f32 ? static_cast<void*>(out_f32) : static_cast<void*>(out_bf16);
  c.dn.out_f32 = out_f32 != nullptr;
  c.dn.n = hidden;
  c.dn.k = inter;
  c.dn.tokens = tokens;
  c.dn.top_k = top_k;
  c.ready = ready;
  c.status = status;
  c.spins = spins;
  bool one = ready != nullptr && status != nullptr && tune_get(kTuneChain) != 1 && slot_chain_fits(c);
  if (one && sel != nullptr)   // the selection inside the launch: one token whose score row fits a wavefront's registers
    one = tokens == 1 && top_k <= kWave && sel->n_experts <= 8 * kWave && tune_get(kTuneSelectAlone) != 1;
  if (one) {
    if (fmt == kFmtFp8F32) {
      one = hidden % 16 == 0 && inter % 16 == 0 && slot_chain_widths_ok<kFmtFp8F32>(hidden, inter);
    } else {
      one = fp4_k_supported(hidden) && fp4_k_compiled(hidden, fp4_group) && fp4_k_supported(inter) &&
            fp4_k_compiled(inter, fp4_group) &&
            (fmt == kFmtNvfp4 ? slot_chain_widths_ok<kFmtNvfp4>(hidden, inter) : slot_chain_widths_ok<kFmtMxfp4>(hidden, inter));
    }
  }
  if (!one) {
    int rc;
    if (sel != nullptr) {   // selection (+ gate/up where that form fits), then the token-major down launch
      if (fmt == kFmtFp8F32)
        rc = dgpp_launch_moe_select_gate_up_swiglu(sel->scores, sel->biased, sel->ids, sel->weights, cfg, tokens, x, x_stride, views,
                                                   inter, hidden, act, act_stride, limit, stream);
      else
        rc = dgpp_launch_moe_select_gate_up_swiglu_fp4(sel->scores, sel->biased, sel->ids, sel->weights, cfg, tokens, x, x_stride,
                                                       views, inter, hidden, act, act_stride, limit, stream, fp4_group);
    } else if (fmt == kFmtFp8F32) {
      rc = dgpp_launch_moe_slot_gate_up_swiglu(x, x_stride, ids, nullptr, views, inter, hidden, 0, 0, nullptr, nullptr, nullptr,
                                               nullptr, act, act_stride, slots, top_k, limit, stream, 7, 7);
    } else {
      rc = dgpp_launch_moe_slot_gate_up_swiglu_fp4(x, x_stride, ids, nullptr, views, inter, hidden, 0, 0, nullptr, nullptr, nullptr,
                                                   nullptr, act, act_stride, slots, top_k, limit, stream, -1, fp4_group, 7, 7);
    }
    if (rc != DGPP_OK) return rc;
    if (fmt == kFmtFp8F32)
      return dgpp_launch_moe_slot_down_accum(act, static_cast<size_t>(act_stride), ids, views, hidden, inter, tokens, top_k,
                                             weights, out_bf16, out_f32, stream);
    return dgpp_launch_moe_slot_down_accum_fp4(act, static_cast<size_t>(act_stride), ids, views, hidden, inter, tokens, top_k,
                                               weights, out_bf16, out_f32, stream, fp4_group);
  }
  return finish(launch_slot_chain(fmt, c, sel, as_stream(stream)), who);
}
// The same with the router's selection inside the launch (one token; more tokens select first and go on as above).
static int select_slot_chain(int fmt, const float* scores, const float* biased, int32_t* ids, float* weights,
                             const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                             const DgppMoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride, float limit,
                             uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status, unsigned spins, void* stream,
                             int fp4_group, const char* who) {
  const int rc = dgpp_moe_config_validate(cfg);
  if (rc != DGPP_OK) return rc;
  if (tokens <= 0) return DGPP_OK;
  if (!scores || !biased || !ids || !weights) return fail_arg(std::string(who) + ": null pointer");
  SelectArgs sel;
  sel.scores = scores;
  sel.biased = biased;
  sel.ids = ids;
  sel.weights = weights;
  sel.mode = cfg->router_mode;
  sel.n_experts = cfg->n_experts;
  sel.scaling = cfg->routed_scaling_factor;
  sel.norm_topk = cfg->norm_topk_prob ? 1 : 0;
  return slot_chain(fmt, x, x_stride, ids, views, inter, hidden, act, act_stride, tokens, cfg->top_k, limit, weights, out_bf16,
                    out_f32, ready, status, spins, stream, fp4_group, who, &sel, cfg);
}
size_t dgpp_moe_slot_chain_ready_bytes(int tokens, int top_k) {
  if (tokens <= 0 || top_k <= 0) return 0;
  return static_cast<size_t>(tokens) * static_cast<size_t>(top_k) * kReadyStride * sizeof(uint32_t);
}
int dgpp_launch_moe_slot_chain(const uint16_t* x, size_t x_stride, const int32_t* ids, const DgppMoeExpertView* views,
                               int inter, int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                               const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                               unsigned spins, void* stream) {
  return slot_chain(kFmtFp8F32, x, x_stride, ids, views, inter, hidden, act, act_stride, tokens, top_k, limit, weights, out_bf16,
                    out_f32, ready, status, spins, stream, 0, "moe_slot_chain");
}
int dgpp_launch_moe_slot_chain_fp4(const uint16_t* x, size_t x_stride, const int32_t* ids, const DgppMoeExpertView* views,
                                   int inter, int hidden, uint16_t* act, int act_stride, int tokens, int top_k, float limit,
                                   const float* weights, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                   unsigned spins, void* stream, int fp4_group) {
  const char* who = "moe_slot_chain_fp4";
  if (fp4_group != 16 && fp4_group != 32) return fail_arg(std::string(who) + ": the fp4 scale group must be 16 or 32");
  return slot_chain(fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4, x, x_stride, ids, views, inter, hidden, act, act_stride, tokens,
                    top_k, limit, weights, out_bf16, out_f32, ready, status, spins, stream, fp4_group, who);
}

int dgpp_launch_moe_select_slot_chain(const float* scores, const float* biased, int32_t* ids, float* weights,
                                      const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                      const DgppMoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride,
                                      float limit, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                      unsigned spins, void* stream) {
  return select_slot_chain(kFmtFp8F32, scores, biased, ids, weights, cfg, tokens, x, x_stride, views, inter, hidden, act, act_stride,
                           limit, out_bf16, out_f32, ready, status, spins, stream, 0, "moe_select_slot_chain");
}
int dgpp_launch_moe_select_slot_chain_fp4(const float* scores, const float* biased, int32_t* ids, float* weights,
                                          const DgppMoeConfig* cfg, int tokens, const uint16_t* x, size_t x_stride,
                                          const DgppMoeExpertView* views, int inter, int hidden, uint16_t* act, int act_stride,
                                          float limit, uint16_t* out_bf16, float* out_f32, uint32_t* ready, int* status,
                                          unsigned spins, void* stream, int fp4_group) {
  const char* who = "moe_select_slot_chain_fp4";
  if (fp4_group != 16 && fp4_group != 32) return fail_arg(std::string(who) + ": the fp4 scale group must be 16 or 32");
  return select_slot_chain(fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4, scores, biased, ids, weights, cfg, tokens, x, x_stride, views,
                           inter, hidden, act, act_stride, limit, out_bf16, out_f32, ready, status, spins, stream, fp4_group, who);
}

// ---- matrix-core launchers (src/kernels/glm_moe_launch.hpp:103-125, :311-345; src/kernels/mma_gemv.hpp:65-85) -----
static int dense_mma(int fmt, const uint16_t* act, size_t act_stride, const MatRef& mat, const float* global, void* out,
                     int out_f32, size_t out_stride, int m, int n, int k, void* ws, size_t ws_bytes, void* stream,
                     const char* who, const uint16_t* act_up = nullptr, float limit = 0.f) {
  if (out_stride == 0) out_stride = static_cast<size_t>(n);
  if (out_stride < static_cast<size_t>(n)) return fail_arg(std::string(who) + ": output row stride narrower than n");
  if ((m + kTileCols - 1) / kTileCols > 65535) return fail_arg(std::string(who) + ": grid dimension overflow");
  DenseArgs a;
  a.act = act;
  a.act_stride = act_stride;
  a.mat = mat;
  a.global = global;
  a.out = out;
  a.out_stride = out_stride;
  a.out_f32 = out_f32;
  a.m = m;
  a.n = n;
  a.k = k;
  a.once = m <= kTileCols;   // one activation tile: one pass over the weights
  a.act_up = act_up;
  a.limit = limit;
  return finish(launch_dense_mma(fmt, a, static_cast<float*>(ws), ws_bytes, as_stream(stream)), who);
}

static int dense_mma_fp8(const uint16_t* act, size_t act_stride, const uint8_t* payload, const void* scales, int e8m0,
                         void* out, int out_f32, int m, int n, int k, size_t out_stride, int rs, int cs, void* ws,
                         size_t ws_bytes, void* stream, const char* who, const uint16_t* act_up = nullptr,
                         float limit = 0.f) {
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (!act || !payload || !scales || !out) return fail_arg(std::string(who) + ": null pointer");
  const bool row_grid = rs == 0 && cs >= 4;
  if (!row_grid && (rs < 4 || rs > 7 || cs < 4 || cs > 7))
    return fail_arg(std::string(who) + ": rs / cs must be 4..7 or a row grid (rs = 0, cs >= 4)");
  if (k <= 0 || !fp8_shape_ok(payload, k))
    return fail_arg(std::string(who) + ": k must be a positive multiple of 16 with a 16-byte aligned payload");
  return dense_mma(e8m0 ? kFmtFp8E8M0 : kFmtFp8F32, act, act_stride, fp8_mat(payload, scales, rs, cs), nullptr, out,
                   out_f32, out_stride, m, n, k, ws, ws_bytes, stream, who, act_up, limit);
}
// The reference's streaming tensor-core GEMV (launch_mma_gemv_fp8{,e8m0}_*) is its decode form for FP8 weights at every
// row count. Here a batch that fits one vector-core pass (up to eight rows) runs on the vector core, which is the
// faster form for it on this chip; from nine rows on the matrix core takes over (ws: its split-K workspace). As with the
// GEMV-named launchers the two cores differ in summation order and meet the same tolerance.
static int mma_gemv_fp8(const uint16_t* act, size_t act_stride, const uint8_t* payload, const void* scales, int e8m0, void* out,
                        int out_f32, int m, int n, int k, size_t out_stride, int rs, int cs, void* ws, size_t ws_bytes,
                        void* stream, const char* who) {
  if (m <= 0 || n <= 0) return DGPP_OK;
  const int fmt = e8m0 ? kFmtFp8E8M0 : kFmtFp8F32;
  if (tune_get(kTuneCore) == 2 || k <= 0 || (tune_get(kTuneCore) != 1 && dense_takes_matrix_core(fmt, m, n, k, ws_bytes, ws != nullptr, 0)))
    return dense_mma_fp8(act, act_stride, payload, scales, e8m0, out, out_f32, m, n, k, out_stride, rs, cs, ws, ws_bytes, stream,
                         who);
  if (!act || !payload || !scales || !out) return fail_arg(std::string(who) + ": null pointer");
  const bool row_grid = rs == 0 && cs >= 4;
  if (!row_grid && (rs < 4 || rs > 7 || cs < 4 || cs > 7))
    return fail_arg(std::string(who) + ": rs / cs must be 4..7 or a row grid (rs = 0, cs >= 4)");
  if (k <= 0 || !fp8_shape_ok(payload, k))
    return fail_arg(std::string(who) + ": k must be a positive multiple of 16 with a 16-byte aligned payload");
  if (out_stride == 0) out_stride = static_cast<size_t>(n);
  if (out_stride < static_cast<size_t>(n)) return fail_arg(std::string(who) + ": output row stride narrower than n");
  return dense_rows(fmt, act, act_stride, fp8_mat(payload, scales, rs, cs), nullptr, out, out_stride, out_f32, m, n, k,
                    as_stream(stream), who, 0, ws, ws_bytes);
}
/* src/kernels/mma_gemv.cu:895-899: the shape the matrix-core GEMV takes. */
int dgpp_mma_gemv_shape_ok(const void* w, const void* act, size_t act_stride, int m, int k) {
  return m >= 1 && k > 0 && (k % 64) == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0 &&
         (reinterpret_cast<uintptr_t>(act) & 15u) == 0 && ((act_stride * 2) % 16) == 0;
}
/* src/kernels/mma_gemv.cu:921-933: whether two projections may share one launch - a decode batch (at most 32 rows), both
 * shapes taken, and a workspace that holds both problems' K-part sums (parts(k) * m * (n0 + n1) floats here). */
int dgpp_mma_gemv_pair_ok(const void* w0, const void* w1, const uint16_t* a0, const uint16_t* a1, size_t act_stride, int m,
                          int n0, int n1, int k, void* ws, size_t ws_bytes) {
  if (!ws || m < 1 || m > 32 || n0 <= 0 || n1 <= 0) return 0;
  if (!dgpp_mma_gemv_shape_ok(w0, a0, act_stride, m, k) || !dgpp_mma_gemv_shape_ok(w1, a1, act_stride, m, k)) return 0;
  const size_t need = static_cast<size_t>(mgeom<kFmtFp8F32>(k).parts) * m * (static_cast<size_t>(n0) + n1) * sizeof(float);
  return need <= ws_bytes;
}
/* src/kernels/mma_gemv.cu:935-961: two FP8 projections of one k and one batch in ONE launch; every row's chain is its
 * single launch's (bitwise dgpp_launch_mma_gemv_fp8_bf16 on each). */
int dgpp_launch_mma_gemv_fp8_bf16_pair(const uint16_t* a0, const uint8_t* w0, const float* s0, uint16_t* o0, int n0,
                                       size_t stride0, const uint16_t* a1, const uint8_t* w1, const float* s1, uint16_t* o1,
                                       int n1, size_t stride1, size_t act_stride, int m, int k, int rs, int cs, void* stream,
                                       void* ws, size_t ws_bytes) {
  const char* who = "mma_gemv_fp8_pair";
  if (m <= 0 || (n0 <= 0 && n1 <= 0)) return DGPP_OK;
  if (n0 <= 0)
    return dgpp_launch_mma_gemv_fp8_bf16(a1, act_stride, w1, s1, o1, m, n1, k, stride1, rs, cs, stream, ws, ws_bytes);
  if (n1 <= 0)
    return dgpp_launch_mma_gemv_fp8_bf16(a0, act_stride, w0, s0, o0, m, n0, k, stride0, rs, cs, stream, ws, ws_bytes);
  if (!a0 || !a1 || !w0 || !w1 || !s0 || !s1 || !o0 || !o1) return fail_arg(std::string(who) + ": null pointer");
  const bool row_grid = rs == 0 && cs >= 4;
  if (!row_grid && (rs < 4 || rs > 7 || cs < 4 || cs > 7))
    return fail_arg(std::string(who) + ": rs / cs must be 4..7 or a row grid (rs = 0, cs >= 4)");
  if (k <= 0 || !fp8_shape_ok(w0, k) || !fp8_shape_ok(w1, k))
    return fail_arg(std::string(who) + ": k must be a positive multiple of 16 with 16-byte aligned payloads");
  if (stride0 == 0) stride0 = static_cast<size_t>(n0);
  if (stride1 == 0) stride1 = static_cast<size_t>(n1);
  if (stride0 < static_cast<size_t>(n0) || stride1 < static_cast<size_t>(n1))
    return fail_arg(std::string(who) + ": output row stride narrower than n");
  if ((m + kTileCols - 1) / kTileCols > 65535) return fail_arg(std::string(who) + ": grid dimension overflow");
  // Each problem takes the core its single launch would take (so that its bits are that launch's): both on the vector
  // core -> one vector-core launch over both; both on the matrix core -> one matrix-core launch; one each -> two launches.
  const int core = tune_get(kTuneCore);
  auto takes_mma = [&](int n) {
    if (core == 2) return true;
    return dense_takes_matrix_core(kFmtFp8F32, m, n, k, ws_bytes, ws != nullptr, 0);
  };
  const bool mma0 = takes_mma(n0), mma1 = takes_mma(n1);
  if (mma0 != mma1 || core == 1) {   // (the bench switch that pins the vector core: the single launchers know how)
    const int rc = dgpp_launch_mma_gemv_fp8_bf16(a0, act_stride, w0, s0, o0, m, n0, k, stride0, rs, cs, stream, ws, ws_bytes);
    if (rc != DGPP_OK) return rc;
    return dgpp_launch_mma_gemv_fp8_bf16(a1, act_stride, w1, s1, o1, m, n1, k, stride1, rs, cs, stream, ws, ws_bytes);
  }
  const bool vector_core = !mma0;
  DenseArgs p[2];
  const uint16_t* acts[2] = {a0, a1};
  const uint8_t* ws_[2] = {w0, w1};
  const float* ss[2] = {s0, s1};
  uint16_t* outs[2] = {o0, o1};
  const int ns[2] = {n0, n1};
  const size_t strides[2] = {stride0, stride1};
  for (int i = 0; i < 2; ++i) {
    p[i].act = acts[i];
    p[i].act_stride = act_stride;
    p[i].mat = fp8_mat(ws_[i], ss[i], rs, cs);
    p[i].global = nullptr;
    p[i].out = outs[i];
    p[i].out_stride = strides[i];
    p[i].out_f32 = 0;
    p[i].m = m;
    p[i].n = ns[i];
    p[i].k = k;
    p[i].once = m <= kTileCols;
  }
  if (vector_core) return finish(launch_dense_multi(kFmtFp8F32, p, 2, as_stream(stream)), who);
  return finish(launch_dense_mma_pair_fp8(p[0], p[1], static_cast<float*>(ws), ws_bytes, as_stream(stream)), who);
}
int dgpp_launch_mma_gemv_fp8_swiglu_f32(const uint16_t* gate, const uint16_t* up, float limit, size_t act_stride,
                                        const uint8_t* w, const float* scales, float* out, int m, int n, int k,
                                        size_t out_stride, int rs, int cs, void* stream) {
  const char* who = "mma_gemv_fp8_swiglu";
  if (m > 0 && n > 0) {
    if (!gate || !up) return fail_arg(std::string(who) + ": null pointer");
    if (((reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up)) & 15u) != 0 || (act_stride & 7u) != 0)
      return fail_arg(std::string(who) + ": gate and up rows must be 16-byte aligned");
  }
  return dense_mma_fp8(gate, act_stride, w, scales, 0, out, 1, m, n, k, out_stride, rs, cs, nullptr, 0, stream, who, up, limit);
}
int dgpp_launch_dense_mma_bf16(const uint16_t* act, size_t act_stride, const uint8_t* payload, const float* scales,
                               uint16_t* out, int m, int n, int k, void* stream, size_t out_stride) {
  return dense_mma_fp8(act, act_stride, payload, scales, 0, out, 0, m, n, k, out_stride, 7, 7, nullptr, 0, stream, "dense_mma");
}
int dgpp_launch_dense_mma_f32(const uint16_t* act, size_t act_stride, const uint8_t* payload, const float* scales,
                              float* out, int m, int n, int k, void* stream, size_t out_stride) {
  return dense_mma_fp8(act, act_stride, payload, scales, 0, out, 1, m, n, k, out_stride, 7, 7, nullptr, 0, stream, "dense_mma");
}
/* src/kernels/scale_gemm.hpp:173-180: the scale GEMM's tile form (many rows against one pass over the weights): here the
 * matrix-core dense form with the scale grid's shifts. */
int dgpp_launch_scale_gemm_tile_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                     const float* w_scales, uint16_t* out, int m, int n, int k, void* stream, int rs, int cs) {
  return dense_mma_fp8(act, act_row_stride_elems, w_payload, w_scales, 0, out, 0, m, n, k, 0, rs, cs, nullptr, 0, stream,
                       "scale_gemm_tile");
}
int dgpp_launch_scale_gemm_tile_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                    const float* w_scales, float* out, int m, int n, int k, void* stream, int rs, int cs) {
  return dense_mma_fp8(act, act_row_stride_elems, w_payload, w_scales, 0, out, 1, m, n, k, 0, rs, cs, nullptr, 0, stream,
                       "scale_gemm_tile");
}
int dgpp_launch_mma_gemv_fp8_bf16(const uint16_t* act, size_t act_stride, const uint8_t* w, const float* scales,
                                  uint16_t* out, int m, int n, int k, size_t out_stride, int rs, int cs, void* stream,
                                  void* ws, size_t ws_bytes) {
  return mma_gemv_fp8(act, act_stride, w, scales, 0, out, 0, m, n, k, out_stride, rs, cs, ws, ws_bytes, stream, "mma_gemv_fp8");
}
int dgpp_launch_mma_gemv_fp8_f32(const uint16_t* act, size_t act_stride, const uint8_t* w, const float* scales, float* out,
                                 int m, int n, int k, size_t out_stride, int rs, int cs, void* stream, void* ws,
                                 size_t ws_bytes) {
  return mma_gemv_fp8(act, act_stride, w, scales, 0, out, 1, m, n, k, out_stride, rs, cs, ws, ws_bytes, stream, "mma_gemv_fp8");
}
int dgpp_launch_mma_gemv_fp8e8m0_bf16(const uint16_t* act, size_t act_stride, const uint8_t* w, const uint8_t* scales,
                                      uint16_t* out, int m, int n, int k, size_t out_stride, int rs, int cs, void* stream,
                                      void* ws, size_t ws_bytes) {
  return mma_gemv_fp8(act, act_stride, w, scales, 1, out, 0, m, n, k, out_stride, rs, cs, ws, ws_bytes, stream,
                       "mma_gemv_fp8e8m0");
}
int dgpp_launch_mma_gemv_fp8e8m0_f32(const uint16_t* act, size_t act_stride, const uint8_t* w, const uint8_t* scales,
                                     float* out, int m, int n, int k, size_t out_stride, int rs, int cs, void* stream,
                                     void* ws, size_t ws_bytes) {
  return mma_gemv_fp8(act, act_stride, w, scales, 1, out, 1, m, n, k, out_stride, rs, cs, ws, ws_bytes, stream,
                       "mma_gemv_fp8e8m0");
}

static int dense_mma_fp4(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, void* out, int out_f32, int m,
                         int n, int k, void* stream, size_t out_stride = 0, void* ws = nullptr, size_t ws_bytes = 0) {
  const char* who = "dense_mma_fp4";
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (!w || !act || !w->payload || !w->scales || !out) return fail_arg(std::string(who) + ": null pointer");
  if (w->scale_group != 16 && w->scale_group != 32)
    return fail_arg(std::string(who) + ": the scale group must be 16 (NVFP4) or 32 (MXFP4)");
  if (w->scale_group == 16 && !w->global_scale) return fail_arg(std::string(who) + ": an NVFP4 matrix needs its global scale");
  if (w->rows < n || w->cols != k) return fail_arg(std::string(who) + ": matrix geometry does not match n, k");
  if (k <= 0 || k % 32 != 0 || !aligned16(w->payload))
    return fail_arg(std::string(who) + ": k must be a multiple of 32 and the payload 16-byte aligned");
  MatRef mat;
  mat.payload = w->payload;
  mat.scales = w->scales;
  mat.divisor = 1.f;
  mat.rs = 0;
  mat.cs = 0;
  return dense_mma(w->scale_group == 16 ? kFmtNvfp4 : kFmtMxfp4, act, act_stride, mat, w->global_scale, out, out_f32,
                   out_stride, m, n, k, ws, ws_bytes, stream, who);
}
int dgpp_launch_mma_gemv_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, uint16_t* out, int m,
                                  int n, int k, size_t out_stride, void* stream, void* ws, size_t ws_bytes) {
  return dense_mma_fp4(act, act_stride, w, out, 0, m, n, k, stream, out_stride, ws, ws_bytes);
}
int dgpp_launch_mma_gemv_fp4_f32(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, float* out, int m, int n,
                                 int k, size_t out_stride, void* stream, void* ws, size_t ws_bytes) {
  return dense_mma_fp4(act, act_stride, w, out, 1, m, n, k, stream, out_stride, ws, ws_bytes);
}
// ---- the entry point that allocates nothing ------------------------------------------------------------------------
// dgpp_launch_mma_gemv_fp4_bf16 with the split-K workspace taken from a file-scope device array instead of a caller's
// buffer, for callers that cannot allocate one (code under graph capture, tight serving loops). Each GPU holds its own
// copy of the array at its own address; the address is looked up once per device and handed to the kernels as an
// ordinary argument (the array's name is only a host-side handle). The partial sums of a call are all written before the
// folding launch reads them, so nothing has to start at zero; calls that overlap on one GPU share the array and race.
}  // extern "C"
namespace {
constexpr size_t kStaticScratchBytes = DGPP_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
namespace {
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {nullptr};
// The stream a device's array is bound to: launches on ONE stream follow each other, launches on two could overlap and
// race on the array, so a second stream is refused until the caller releases the binding (dgpp_static_scratch_release,
// after it has made sure the bound stream's work is done).
void* g_scratch_stream[kMaxDevices] = {nullptr};
bool g_scratch_bound[kMaxDevices] = {false};
inline bool dense_mma_would_split(int parts, int m, int n) { return dense_mfma_would_split(parts, m, n); }
// The device address of `scratch` on the current device (looked up on the first call there), bound to `stream`.
int static_scratch(void** ptr, void* stream, const char* who) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return finish(err, who);
  if (device < 0 || device >= kMaxDevices) return fail_arg(std::string(who) + ": device ordinal beyond the per-device table");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[device] == nullptr) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return finish(err, who);
    if (p == nullptr) return fail_arg(std::string(who) + ": the scratch array has no address on this device");
    g_scratch_ptr[device] = p;
  }
  if (g_scratch_bound[device] && g_scratch_stream[device] != stream)
    return fail_arg(std::string(who) + ": the static workspace of this device is in use by another stream (calls that "
                    "overlap would race on it); finish that stream's work and call dgpp_static_scratch_release first");
  g_scratch_bound[device] = true;
  g_scratch_stream[device] = stream;
  *ptr = g_scratch_ptr[device];
  return DGPP_OK;
}
}  // namespace
extern "C" {
int dgpp_launch_mma_gemv_fp4_bf16_static(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, uint16_t* out,
                                         int m, int n, int k, size_t out_stride, void* stream) {
  const char* who = "mma_gemv_fp4_static";
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (k <= 0 || k % 32 != 0) return fail_arg(std::string(who) + ": k must be a positive multiple of 32");
  const int parts = w && w->scale_group == 32 ? mgeom<kFmtMxfp4>(k).parts : mgeom<kFmtNvfp4>(k).parts;
  // Only the split form uses the workspace: a launch that would run unsplit anyway (one part, or row tiles that fill
  // the chip by themselves) needs none and is never refused for its size.
  if (!dense_mma_would_split(parts, m, n)) return dense_mma_fp4(act, act_stride, w, out, 0, m, n, k, stream, out_stride, nullptr, 0);
  const size_t need = static_cast<size_t>(parts) * static_cast<size_t>(m) * static_cast<size_t>(n) * sizeof(float);
  if (need > kStaticScratchBytes)
    return fail_arg(std::string(who) + ": parts(k) * m * n floats (" + std::to_string(need) + " bytes) exceed the " +
                    std::to_string(kStaticScratchBytes) + "-byte static workspace; pass a workspace of your own to "
                    "dgpp_launch_mma_gemv_fp4_bf16");
  void* ws = nullptr;
  const int rc = static_scratch(&ws, stream, who);
  if (rc != DGPP_OK) return rc;
  return dense_mma_fp4(act, act_stride, w, out, 0, m, n, k, stream, out_stride, ws, kStaticScratchBytes);
}
int dgpp_static_scratch_release(void) {
  int device = -1;
  const hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return finish(err, "static_scratch_release");
  if (device < 0 || device >= kMaxDevices) return fail_arg("static_scratch_release: device ordinal beyond the per-device table");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  g_scratch_bound[device] = false;
  return DGPP_OK;
}
int dgpp_launch_dense_mma_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, uint16_t* out, int m,
                                   int n, int k, void* stream) {
  return dense_mma_fp4(act, act_stride, w, out, 0, m, n, k, stream);
}
int dgpp_launch_dense_mma_fp4_f32(const uint16_t* act, size_t act_stride, const DgppFp4Matrix* w, float* out, int m, int n,
                                  int k, void* stream) {
  return dense_mma_fp4(act, act_stride, w, out, 1, m, n, k, stream);
}

static int grouped_mma_fp8(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs, int max_rows,
                           int rows_per_block, const DgppMoeExpertView* views, int which, void* out, int out_f32,
                           size_t out_stride, int n, int k, void* stream, const int32_t* act_rows,
                           const float* gate_up_limit = nullptr) {
  const char* who = "moe grouped mma";
  if (n_segs <= 0 || n <= 0) return DGPP_OK;
  if (!act || !segs || !views || !out) return fail_arg(std::string(who) + ": null pointer");
  if (k <= 0 || k % 16 != 0) return fail_arg(std::string(who) + ": k must be a positive multiple of 16");
  return grouped(kFmtFp8F32, act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, out_f32,
                 out_stride, n, k, stream, who, true, act_rows, gate_up_limit);
}
int dgpp_launch_moe_grouped_mma_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                     int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                     uint16_t* out, size_t out_stride, int n, int k, void* stream,
                                     const int32_t* act_rows) {
  return grouped_mma_fp8(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 0, out_stride, n, k,
                         stream, act_rows);
}
int dgpp_launch_moe_grouped_mma_f32(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                    int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which, float* out,
                                    size_t out_stride, int n, int k, void* stream, const int32_t* act_rows) {
  return grouped_mma_fp8(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 1, out_stride, n, k,
                         stream, act_rows);
}
static int grouped_mma_fp4(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs, int max_rows,
                           int rows_per_block, const DgppMoeExpertView* views, int which, void* out, int out_f32,
                           size_t out_stride, int n, int k, void* stream, const int32_t* act_rows, int fp4_group,
                           const float* gate_up_limit = nullptr, void* out_up = nullptr) {
  const char* who = "moe grouped mma fp4";
  if (n_segs <= 0 || n <= 0) return DGPP_OK;
  if (!act || !segs || !views || !out) return fail_arg(std::string(who) + ": null pointer");
  if (fp4_group != 16 && fp4_group != 32) return fail_arg(std::string(who) + ": the fp4 scale group must be 16 or 32");
  if (k <= 0 || k % 32 != 0) return fail_arg(std::string(who) + ": k must be a positive multiple of 32");
  return grouped(fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4, act, act_stride, segs, n_segs, max_rows, rows_per_block, views,
                 which, out, out_f32, out_stride, n, k, stream, who, true, act_rows, gate_up_limit, out_up);
}
/* src/kernels/glm_moe.cu:4809-4823: one segment read from the device, the grouped kernel's chain. */
int dgpp_launch_dense_mma_fp4_prod_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* seg,
                                        const DgppMoeExpertView* views, int which, uint16_t* out, int m, int n, int k,
                                        void* stream, int fp4_group) {
  if (m <= 0 || n <= 0) return DGPP_OK;
  return grouped_mma_fp4(act, act_stride, seg, 1, m, 0, views, which, out, 0, static_cast<size_t>(n), n, k, stream, nullptr,
                         fp4_group);
}
/* src/kernels/dense_fp4_decode.cu:297-308: the small dense NVFP4 shard form. The shape rule is the reference's (one
 * 16-row tile, n and k up to 17408, k in whole 128-element steps); the launch is the production form's, whose bits the
 * reference's decode form shares. *launched = 0 and nothing runs when the shape is outside the rule. */
int dgpp_dense_fp4_decode_shape(int m, int n, int k, int fp4_group) {
  return fp4_group == 16 && m > 0 && m <= 16 && n > 0 && n <= 17408 && k > 0 && k <= 17408 && k % 128 == 0;
}
int dgpp_try_dense_fp4_decode_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* seg,
                                   const DgppMoeExpertView* views, int which, uint16_t* out, int m, int n, int k,
                                   void* stream, int fp4_group, int* launched) {
  if (launched) *launched = 0;
  if (!dgpp_dense_fp4_decode_shape(m, n, k, fp4_group)) return DGPP_OK;
  const int rc = dgpp_launch_dense_mma_fp4_prod_bf16(act, act_stride, seg, views, which, out, m, n, k, stream, fp4_group);
  if (rc == DGPP_OK && launched) *launched = 1;
  return rc;
}
/* src/kernels/dense_fp4_decode.cu:310-319: gate and up of one segment; one launch here, the bits of two prod launches. */
int dgpp_launch_dense_mma_fp4_gate_up_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* seg,
                                           const DgppMoeExpertView* views, uint16_t* gate, uint16_t* up, int m, int n,
                                           int k, void* stream, int fp4_group) {
  if (m <= 0 || n <= 0) return DGPP_OK;
  if (!up) return fail_arg("dense mma fp4 gate_up: null pointer");
  return grouped_mma_fp4(act, act_stride, seg, 1, m, 0, views, 0, gate, 0, static_cast<size_t>(n), n, k, stream, nullptr,
                         fp4_group, nullptr, up);
}
int dgpp_launch_moe_grouped_mma_gate_up_swiglu(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs,
                                               int n_segs, int max_rows, int rows_per_block, const DgppMoeExpertView* views,
                                               uint16_t* out, size_t out_stride, int n, int k, float limit, void* stream,
                                               const int32_t* act_rows) {
  return grouped_mma_fp8(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, 0, out, 0, out_stride, n, k, stream,
                         act_rows, &limit);
}
int dgpp_launch_moe_grouped_mma_gate_up_swiglu_fp4(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs,
                                                   int n_segs, int max_rows, int rows_per_block,
                                                   const DgppMoeExpertView* views, uint16_t* out, size_t out_stride, int n,
                                                   int k, float limit, void* stream, const int32_t* act_rows,
                                                   int fp4_group) {
  return grouped_mma_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, 0, out, 0, out_stride, n, k, stream,
                         act_rows, fp4_group, &limit);
}
int dgpp_launch_moe_grouped_mma_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                         int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                         uint16_t* out, size_t out_stride, int n, int k, void* stream,
                                         const int32_t* act_rows, int fp4_group, int tile_rows) {
  (void)tile_rows;   // the reference's activation ring depth; one 16-row tile per weight pass here
  return grouped_mma_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 0, out_stride, n, k,
                         stream, act_rows, fp4_group);
}
int dgpp_launch_moe_grouped_mma_fp4_f32(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                        int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                        float* out, size_t out_stride, int n, int k, void* stream, const int32_t* act_rows,
                                        int fp4_group, int tile_rows) {
  (void)tile_rows;
  return grouped_mma_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 1, out_stride, n, k,
                         stream, act_rows, fp4_group);
}

static int grouped_fp8(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs, int max_rows,
                       int rows_per_block, const DgppMoeExpertView* views, int which, void* out, int out_f32,
                       size_t out_stride, int n, int k, void* stream) {
  // src/kernels/glm_moe.cu:1062-1090
  const char* who = "moe grouped gemv";
  if (n_segs <= 0 || n <= 0) return DGPP_OK;
  if (!act || !segs || !views || !out) return fail_arg(std::string(who) + ": null pointer");
  if (k <= 0 || k % 16 != 0) return fail_arg(std::string(who) + ": k must be a positive multiple of 16");
  if (stage_bytes(1, k) > kMaxLdsBytes) return fail_arg(std::string(who) + ": k exceeds the smem budget");
  return grouped(kFmtFp8F32, act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, out_f32,
                 out_stride, n, k, stream, who);
}
int dgpp_launch_moe_grouped_gemv_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                      int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                      uint16_t* out, size_t out_stride, int n, int k, void* stream) {
  return grouped_fp8(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 0, out_stride, n, k, stream);
}
int dgpp_launch_moe_grouped_gemv_f32(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                     int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                     float* out, size_t out_stride, int n, int k, void* stream) {
  return grouped_fp8(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 1, out_stride, n, k, stream);
}

static int grouped_fp4(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs, int max_rows,
                       int rows_per_block, const DgppMoeExpertView* views, int which, void* out, int out_f32,
                       size_t out_stride, int n, int k, void* stream, int fp4_group) {
  // src/kernels/glm_moe.cu:2231-2266
  const char* who = "moe grouped gemv fp4";
  if (n_segs <= 0 || n <= 0) return DGPP_OK;
  if (!act || !segs || !views || !out) return fail_arg(std::string(who) + ": null pointer");
  if (fp4_group != 16 && fp4_group != 32) return fail_arg(std::string(who) + ": the fp4 scale group must be 16 or 32");
  if (!fp4_k_supported(k) || !fp4_k_compiled(k, fp4_group))
    return fail_arg(std::string(who) + ": k must be a multiple of 32 in the fp4 core's compiled set");
  return grouped(fp4_group == 16 ? kFmtNvfp4 : kFmtMxfp4, act, act_stride, segs, n_segs, max_rows, rows_per_block, views,
                 which, out, out_f32, out_stride, n, k, stream, who);
}
int dgpp_launch_moe_grouped_gemv_fp4_bf16(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs,
                                          int n_segs, int max_rows, int rows_per_block, const DgppMoeExpertView* views,
                                          int which, uint16_t* out, size_t out_stride, int n, int k, void* stream,
                                          int fp4_group) {
  return grouped_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 0, out_stride, n, k,
                     stream, fp4_group);
}
int dgpp_launch_moe_grouped_gemv_fp4_f32(const uint16_t* act, size_t act_stride, const DgppMoeSegment* segs, int n_segs,
                                         int max_rows, int rows_per_block, const DgppMoeExpertView* views, int which,
                                         float* out, size_t out_stride, int n, int k, void* stream, int fp4_group) {
  return grouped_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, 1, out_stride, n, k,
                     stream, fp4_group);
}

int dgpp_launch_fp4_gemv_bf16(const uint16_t* act, size_t act_row_stride_elems, const DgppFp4Matrix* w, uint16_t* out,
                              int m, int n, int k, void* stream) {
  return fp4_gemv(act, act_row_stride_elems, w, out, 0, m, n, k, stream);
}
int dgpp_launch_fp4_gemv_f32(const uint16_t* act, size_t act_row_stride_elems, const DgppFp4Matrix* w, float* out,
                             int m, int n, int k, void* stream) {
  return fp4_gemv(act, act_row_stride_elems, w, out, 1, m, n, k, stream);
}
int dgpp_fp4_gemv_accepts(const DgppFp4Matrix* w) {
  // src/kernels/fp4_gemv.cu:97-102
  return w && w->payload && w->scales && (w->scale_group == 32 || w->global_scale) && w->cols > 0 && w->cols <= 16384 &&
                 fp4_k_supported(static_cast<int>(w->cols)) && aligned16(w->payload) &&
                 (w->scale_group == 16 || w->scale_group == 32) &&
                 fp4_k_compiled(static_cast<int>(w->cols), w->scale_group)
             ? 1
             : 0;
}

int dgpp_launch_scale_gemm_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                const float* w_scales, uint16_t* out, int m, int n, int k, void* stream,
                                size_t out_row_stride_elems, int mma_from_rows, void* ws, size_t ws_bytes) {
  return scale_gemm(act, act_row_stride_elems, w_payload, w_scales, 0, out, 0, m, n, k, stream, out_row_stride_elems, 7,
                    7, 0, -1, false, "scale_gemm", mma_from_rows, ws, ws_bytes);
}
int dgpp_launch_scale_gemm_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                               const float* w_scales, float* out, int m, int n, int k, void* stream,
                               size_t out_row_stride_elems, int mma_from_rows, int last_row_only, void* ws,
                               size_t ws_bytes, int compact_row) {
  return scale_gemm(act, act_row_stride_elems, w_payload, w_scales, 0, out, 1, m, n, k, stream, out_row_stride_elems, 7,
                    7, last_row_only, compact_row, false, "scale_gemm", mma_from_rows, ws, ws_bytes);
}
int dgpp_launch_scale_gemm_grid_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                     const float* w_scales, uint16_t* out, int m, int n, int k, void* stream,
                                     size_t out_row_stride_elems, int rs, int cs, int decode_mma, void* ws,
                                     size_t ws_bytes, int prefill_tile) {
  (void)decode_mma; (void)prefill_tile;
  return scale_gemm(act, act_row_stride_elems, w_payload, w_scales, 0, out, 0, m, n, k, stream, out_row_stride_elems, rs,
                    cs, 0, -1, true, "scale_gemm_grid", 0, ws, ws_bytes);
}
int dgpp_launch_scale_gemm_grid_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                    const float* w_scales, float* out, int m, int n, int k, void* stream,
                                    size_t out_row_stride_elems, int rs, int cs, int decode_mma, void* ws,
                                    size_t ws_bytes, int prefill_tile) {
  (void)decode_mma; (void)prefill_tile;
  return scale_gemm(act, act_row_stride_elems, w_payload, w_scales, 0, out, 1, m, n, k, stream, out_row_stride_elems, rs,
                    cs, 0, -1, true, "scale_gemm_grid", 0, ws, ws_bytes);
}
int dgpp_launch_scale_gemm_grid_e8m0_bf16(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                          const uint8_t* w_scales, uint16_t* out, int m, int n, int k, void* stream,
                                          size_t out_row_stride_elems, int rs, int cs, void* ws, size_t ws_bytes,
                                          int prefill_tile) {
  (void)prefill_tile;
  return scale_gemm(act, act_row_stride_elems, w_payload, w_scales, 1, out, 0, m, n, k, stream, out_row_stride_elems, rs,
                    cs, 0, -1, true, "scale_gemm_grid_e8m0", 0, ws, ws_bytes);
}
int dgpp_launch_scale_gemm_grid_e8m0_f32(const uint16_t* act, size_t act_row_stride_elems, const uint8_t* w_payload,
                                         const uint8_t* w_scales, float* out, int m, int n, int k, void* stream,
                                         size_t out_row_stride_elems, int rs, int cs, void* ws, size_t ws_bytes,
                                         int prefill_tile) {
  (void)prefill_tile;
  return scale_gemm(act, act_row_stride_elems, w_payload, w_scales, 1, out, 1, m, n, k, stream, out_row_stride_elems, rs,
                    cs, 0, -1, true, "scale_gemm_grid_e8m0", 0, ws, ws_bytes);
}

int dgpp_launch_scale_gemv_multi_bf16(const DgppFp8GemvProblem* problems, int n_problems, const uint16_t* act,
                                      size_t act_row_stride_elems, int rows, int k, void* stream) {
  // src/kernels/scale_gemm.cu:625-672: each problem's output is bitwise the single launcher's.
  const char* who = "scale_gemv_multi";
  if (n_problems <= 0 || rows <= 0) return DGPP_OK;
  if (!problems || !act) return fail_arg(std::string(who) + ": null pointer");
  if (n_problems > 4) return fail_arg(std::string(who) + ": at most four problems");
  if (rows > kMaxActRows) return fail_arg(std::string(who) + ": at most eight rows");
  for (int i = 0; i < n_problems; ++i) {
    const DgppFp8GemvProblem& p = problems[i];
    if (p.bf16_weight) return fail_arg(std::string(who) + ": bf16 problems are outside this library's path");
    if (!p.payload || !p.scales || !p.out || p.n <= 0) return fail_arg(std::string(who) + ": null pointer");
    if (!fp8_shape_ok(p.payload, k)) return fail_arg(std::string(who) + ": k must be a multiple of 16 with aligned payloads");
  }
  // One launch over all problems' row tiles where the rows fit one stage (the decode case); otherwise one launch each.
  if (tune_get(kTuneCore) != 2 && rows <= max_stage_rows(k)) {
    DenseArgs d[kMaxDenseProblems];
    for (int i = 0; i < n_problems; ++i) {
      const DgppFp8GemvProblem& p = problems[i];
      const size_t out_stride = p.out_stride ? p.out_stride : static_cast<size_t>(p.n);
      if (out_stride < static_cast<size_t>(p.n)) return fail_arg(std::string(who) + ": output row stride narrower than n");
      d[i].act = act;
      d[i].act_stride = act_row_stride_elems;
      d[i].mat = fp8_mat(p.payload, p.scales, p.rs, p.cs);
      d[i].global = nullptr;
      d[i].out = p.out;
      d[i].out_stride = out_stride;
      d[i].out_f32 = 0;
      d[i].m = rows;
      d[i].n = p.n;
      d[i].k = k;
      d[i].once = 1;
    }
    return finish(launch_dense_multi(kFmtFp8F32, d, n_problems, as_stream(stream)), who);
  }
  for (int i = 0; i < n_problems; ++i) {
    const DgppFp8GemvProblem& p = problems[i];
    const int rc = scale_gemm(act, act_row_stride_elems, p.payload, p.scales, 0, p.out, 0, rows, p.n, k, stream,
                              p.out_stride, p.rs, p.cs, 0, -1, false, who);
    if (rc != DGPP_OK) return rc;
  }
  return DGPP_OK;
}

int dgpp_fp8_gemv_can_stage(const void* w_payload, int k) { return fp8_shape_ok(w_payload, k) ? 1 : 0; }

static int fp8_dequant(const uint8_t* payload, const void* scales, int e8m0, uint16_t* out, int64_t rows, int64_t cols,
                       void* stream, int rs, int cs) {
  // src/kernels/fp8_dequant.cu:52-72
  if (rows <= 0 || cols <= 0) return fail_arg("fp8_dequant: rows and cols must be positive");
  if (!payload || !scales || !out) return fail_arg("fp8_dequant: null pointer");
  if (rs < 0 || cs < 4 || rs > 30 || cs > 30) return fail_arg("fp8_dequant: rs must be non-negative, cs >= 4");
  if ((rows * cols + 255) / 256 > 2147483647LL) {
    g_last_error = "fp8_dequant: grid too large";
    return DGPP_RUNTIME_ERROR;
  }
  return finish(run_fp8_dequant(payload, scales, e8m0, out, rows, cols, rs, cs, as_stream(stream)), "fp8_dequant");
}
int dgpp_launch_fp8_dequant_blocks(const uint8_t* payload, const float* scales, uint16_t* out_bf16, int64_t rows,
                                   int64_t cols, void* stream, int rs, int cs) {
  return fp8_dequant(payload, scales, 0, out_bf16, rows, cols, stream, rs, cs);
}
int dgpp_launch_fp8_dequant_blocks_e8m0(const uint8_t* payload, const uint8_t* scales, uint16_t* out_bf16, int64_t rows,
                                        int64_t cols, void* stream, int rs, int cs) {
  return fp8_dequant(payload, scales, 1, out_bf16, rows, cols, stream, rs, cs);
}

}  // extern "C"
