// A bound MoE layer made resident in one call: the tensors a *_bind_layer call found in the checkpoint's shards are
// cut to this rank's slice of the intermediate dimension (gate / up rows [rank * M, (rank + 1) * M), the matching
// columns of down, M = inter / world), uploaded into ONE device allocation, described by an expert table and handed
// to the layer driver. Reference counterpart: the resident build of a GLM MoE layer,
// src/models/glm/loader.cpp:418-471 (build_moe: router, shared expert, every routed expert sliced like the shared
// one, NVFP4 globals gathered into one array) with the slicing rules of src/models/quant_matrix.hpp:67-96, 140-164.
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/dgpp_amd_layer.h"
#include "../../include/dgpp_amd_loader.h"

struct DgppMoeResident {
  void* arena = nullptr;
  size_t bytes = 0;
  DgppMoeLayer* layer = nullptr;
  DgppMoeConfig cfg{};   // the rank's geometry (inter = M)
  int32_t shared_inter = 0;
};

namespace {

thread_local std::string g_resident_error;

struct Refused : std::runtime_error {
  int code;
  Refused(int c, const std::string& what) : std::runtime_error(what), code(c) {}
};
[[noreturn]] void refuse(const std::string& what) { throw Refused(DGPP_INVALID_ARGUMENT, "moe_resident_load: " + what); }
void loader_ok(int rc) {
  if (rc != DGPP_OK) throw Refused(rc, std::string("moe_resident_load: ") + dgpp_loader_last_error());
}
void hip_ok(hipError_t e, const char* what) {
  if (e != hipSuccess) throw Refused(DGPP_RUNTIME_ERROR, std::string("moe_resident_load: ") + what + ": " + hipGetErrorString(e));
}
size_t up256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

enum class Kind { Fp8, Fp4, Mxfp8 };
Kind kind_of(int format) {
  switch (format) {
    case DGPP_BIND_FP8:
    case DGPP_BIND_FP8_BF16_SCALES: return Kind::Fp8;
    case DGPP_BIND_NVFP4:
    case DGPP_BIND_NVFP4_MODELOPT:
    case DGPP_BIND_NVFP4_COMPRESSED:
    case DGPP_BIND_MXFP4: return Kind::Fp4;
    case DGPP_BIND_MXFP8:
    case DGPP_BIND_MXFP8_SCALE_INV: return Kind::Mxfp8;
    default: refuse("unknown tensor format " + std::to_string(format));
  }
}
int fp4_group_of(int format) { return format == DGPP_BIND_MXFP4 ? 32 : 16; }

// One matrix's slice: axis 0 = rows [start, start + count), axis 1 = columns; whole = no cut at all.
struct Cut {
  int axis;
  int64_t start, count;
  bool whole;
};

// The logical shape of a bound matrix (FP4 payloads hold two columns per byte).
void logical_shape(const DgppMoeMatrixTensors& t, int64_t& rows, int64_t& cols) {
  if (t.payload.rank != 2) refuse("a weight payload must be a matrix");
  rows = t.payload.shape[0];
  cols = kind_of(t.format) == Kind::Fp4 ? t.payload.shape[1] * 2 : t.payload.shape[1];
}

struct Sizes {
  size_t payload, scales;
};
Sizes sliced_sizes(const DgppMoeMatrixTensors& t, const Cut& c) {
  int64_t rows, cols;
  logical_shape(t, rows, cols);
  const int64_t r = c.whole || c.axis == 1 ? rows : c.count, k = c.whole || c.axis == 0 ? cols : c.count;
  switch (kind_of(t.format)) {
    case Kind::Fp8: {
      if (c.whole) return {static_cast<size_t>(rows * cols), static_cast<size_t>(((rows + 127) / 128) * ((cols + 127) / 128)) * 4};
      DgppQuantMatrix m{nullptr, nullptr, nullptr, rows, cols, 128, 128};
      const int64_t n = dgpp_quant_slice_scale_count(&m, c.axis, c.start, c.count);
      if (n < 0) refuse("the rank's slice does not re-block to a scale grid the launchers take (gcd(128, start, count) must be a power of two >= 32)");
      return {static_cast<size_t>(r * k), static_cast<size_t>(n) * 4};
    }
    case Kind::Fp4: {
      const int g = fp4_group_of(t.format);
      if (k % g != 0) refuse("an FP4 slice must hold whole scale groups");
      return {static_cast<size_t>(r * (k / 2)), static_cast<size_t>(r * (k / g))};
    }
    default:
      if (k % 32 != 0) refuse("an MXFP8 slice must hold whole 32-column scale blocks");
      return {static_cast<size_t>(r * k), static_cast<size_t>(r * (k / 32))};
  }
}

struct Bump {
  uint8_t* base = nullptr;
  size_t used = 0, cap = 0;
  uint8_t* take(size_t bytes) {
    const size_t at = used;
    used += up256(bytes);
    if (base && used > cap) throw Refused(DGPP_RUNTIME_ERROR, "moe_resident_load: arena accounting");
    return base ? base + at : nullptr;
  }
};

struct DeviceMatrix {
  const uint8_t* payload = nullptr;
  const uint8_t* scales = nullptr;   // F32 grid, e4m3 / e8m0 bytes
  int64_t rows = 0, cols = 0;
  int block_rows = 128, block_cols = 128;   // FP8 grid after the cut
};

void to_device(uint8_t* dst, const void* src, size_t bytes) {
  if (bytes) hip_ok(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "upload");
}

// Cuts and uploads one matrix (dry: only the arena's accounting advances).
DeviceMatrix place(const DgppMoeMatrixTensors& t, const Cut& c, Bump& bump, bool dry) {
  int64_t rows, cols;
  logical_shape(t, rows, cols);
  const Sizes sz = sliced_sizes(t, c);
  DeviceMatrix d;
  d.rows = c.whole || c.axis == 1 ? rows : c.count;
  d.cols = c.whole || c.axis == 0 ? cols : c.count;
  uint8_t* p_dev = bump.take(sz.payload);
  uint8_t* s_dev = bump.take(sz.scales);
  d.payload = p_dev;
  d.scales = s_dev;
  const Kind kind = kind_of(t.format);
  if (kind == Kind::Fp8 && !c.whole) {   // the grid of the cut, known without touching the data
    int64_t g = 128;   // gcd(block, start, count): dgpp_quant_slice's rule
    for (int64_t v : {c.start, c.count}) {
      int64_t a = g, b = v;
      while (b != 0) {
        const int64_t r = a % b;
        a = b;
        b = r;
      }
      g = a;
    }
    (c.axis == 0 ? d.block_rows : d.block_cols) = static_cast<int>(g);
  }
  if (dry) return d;
  if (!t.payload.data || !t.scales.data) refuse("a bound tensor has no data");
  {
    // The copies below read whole rows of the UNSLICED tensors at sizes derived from the payload's shape: a
    // description whose byte counts do not cover them (hand-filled, or inconsistent) is refused before any read.
    const Kind whole_kind = kind_of(t.format);
    uint64_t need_payload, need_scales;
    if (whole_kind == Kind::Fp8) {
      need_payload = static_cast<uint64_t>(rows) * static_cast<uint64_t>(cols);
      need_scales = static_cast<uint64_t>((rows + 127) / 128) * static_cast<uint64_t>((cols + 127) / 128) *
                    (t.format == DGPP_BIND_FP8_BF16_SCALES ? 2u : 4u);
    } else {
      const int64_t group = whole_kind == Kind::Fp4 ? fp4_group_of(t.format) : 32;
      need_payload = static_cast<uint64_t>(rows) * static_cast<uint64_t>(whole_kind == Kind::Fp4 ? cols / 2 : cols);
      need_scales = static_cast<uint64_t>(rows) * static_cast<uint64_t>(cols / group);
    }
    if (rows <= 0 || cols <= 0 || t.payload.nbytes < need_payload || t.scales.nbytes < need_scales)
      refuse("a bound tensor's byte count does not cover the matrix its shape describes");
  }
  const uint8_t* payload = static_cast<const uint8_t*>(t.payload.data);
  const uint8_t* scales = static_cast<const uint8_t*>(t.scales.data);
  if (kind == Kind::Fp8) {
    const int64_t grid = ((rows + 127) / 128) * ((cols + 127) / 128);
    std::vector<float> wide;   // a BF16 grid widened (exact); an F32 grid copied out of the (unaligned) mapping when cut
    const bool bf16 = t.format == DGPP_BIND_FP8_BF16_SCALES;
    if (bf16 || !c.whole) {
      wide.resize(static_cast<size_t>(grid));
      if (bf16) {
        for (int64_t i = 0; i < grid; ++i) {
          uint16_t b;
          std::memcpy(&b, scales + i * 2, 2);
          const uint32_t u = static_cast<uint32_t>(b) << 16;
          std::memcpy(&wide[static_cast<size_t>(i)], &u, 4);
        }
      } else {
        std::memcpy(wide.data(), scales, static_cast<size_t>(grid) * 4);
      }
    }
    if (c.whole) {
      to_device(p_dev, payload, sz.payload);
      to_device(s_dev, bf16 ? static_cast<const void*>(wide.data()) : static_cast<const void*>(scales), sz.scales);
      return d;
    }
    DgppQuantMatrix whole{payload, wide.data(), nullptr, rows, cols, 128, 128}, cut{};
    std::vector<uint8_t> pbuf(sz.payload);
    std::vector<float> sbuf(sz.scales / 4);
    loader_ok(dgpp_quant_slice(&whole, c.axis, c.start, c.count, pbuf.data(), sbuf.data(), &cut));
    if (cut.scale_block_rows != d.block_rows || cut.scale_block_cols != d.block_cols)
      throw Refused(DGPP_RUNTIME_ERROR, "moe_resident_load: scale grid accounting");
    to_device(p_dev, pbuf.data(), sz.payload);
    to_device(s_dev, sbuf.data(), sz.scales);
    return d;
  }
  // FP4 and MXFP8: scale bytes per row, `per` columns per scale byte, `pack` columns per payload byte
  const int per = kind == Kind::Fp4 ? fp4_group_of(t.format) : 32, pack = kind == Kind::Fp4 ? 2 : 1;
  if (c.whole || c.axis == 0) {   // whole rows are contiguous in the file
    const int64_t r0 = c.whole ? 0 : c.start;
    to_device(p_dev, payload + r0 * (cols / pack), sz.payload);
    to_device(s_dev, scales + r0 * (cols / per), sz.scales);
    return d;
  }
  if (c.start % per != 0) refuse("a column slice must start on a scale-block boundary");
  std::vector<uint8_t> pbuf(sz.payload), sbuf(sz.scales);
  const int64_t src_p = cols / pack, dst_p = c.count / pack, src_s = cols / per, dst_s = c.count / per;
  for (int64_t r = 0; r < rows; ++r) {
    std::memcpy(pbuf.data() + r * dst_p, payload + r * src_p + c.start / pack, static_cast<size_t>(dst_p));
    std::memcpy(sbuf.data() + r * dst_s, scales + r * src_s + c.start / per, static_cast<size_t>(dst_s));
  }
  to_device(p_dev, pbuf.data(), sz.payload);
  to_device(s_dev, sbuf.data(), sz.scales);
  return d;
}

// The kernels DIVIDE a finished NVFP4 dot by the matrix's global: the divisor itself in the engine's own and the
// compressed-tensors spelling, its reciprocal in the ModelOpt one.
float nvfp4_divisor(const DgppMoeMatrixTensors& t) {
  if (!t.global.data || t.global.numel != 1 || t.global.dtype != DGPP_DT_F32) refuse("an NVFP4 matrix needs its F32 global scale");
  float v;
  std::memcpy(&v, t.global.data, 4);
  return t.format == DGPP_BIND_NVFP4_MODELOPT ? 1.0f / v : v;
}

int shift_of(int block) {
  int s = 0;
  while ((1 << s) < block) ++s;
  if ((1 << s) != block) refuse("a scale block must be a power of two");
  return s;
}

void load(const DgppMoeResidentDesc& d, DgppMoeResident& out) {
  if (!d.routed) refuse("null routed tensors");
  if (d.world <= 0 || d.rank < 0 || d.rank >= d.world) refuse("rank must lie in [0, world)");
  const int E = d.cfg.n_experts;
  if (E <= 0 || d.cfg.inter <= 0 || d.cfg.hidden <= 0) refuse("geometry must be positive");
  if (d.cfg.inter % d.world != 0 || d.shared_inter % d.world != 0) refuse("the intermediate dimension must divide by world");
  const int64_t M = d.cfg.inter / d.world, SM = d.shared_inter / d.world;
  const bool whole = d.world == 1;
  const Kind routed_kind = kind_of(d.routed[0].format);
  if (routed_kind == Kind::Mxfp8) refuse("routed experts are block FP8, NVFP4 or MXFP4");
  for (int i = 0; i < E * 3; ++i) {
    if (d.routed[i].format != d.routed[0].format) refuse("one format across the routed experts");
    int64_t r, c;
    logical_shape(d.routed[i], r, c);
    const bool down = i % 3 == 2;
    if (r != (down ? d.cfg.hidden : d.cfg.inter) || c != (down ? d.cfg.inter : d.cfg.hidden))
      refuse("routed matrix " + std::to_string(i) + " does not have the layer's geometry");
  }
  const bool fp4 = routed_kind == Kind::Fp4;
  const bool nvfp4 = fp4 && fp4_group_of(d.routed[0].format) == 16;
  // the shared expert's form
  enum class Shared { None, Fp8Args, Fp4Table, Mxfp8Dense } sh = Shared::None;
  if (d.shared && d.shared_inter > 0) {
    const Kind k = kind_of(d.shared[0].format);
    for (int i = 0; i < 3; ++i) {
      if (d.shared[i].format != d.shared[0].format) refuse("one format across the shared expert's matrices");
      int64_t r, c;
      logical_shape(d.shared[i], r, c);
      if (r != (i == 2 ? d.cfg.hidden : d.shared_inter) || c != (i == 2 ? d.shared_inter : d.cfg.hidden))
        refuse("shared matrix " + std::to_string(i) + " does not have the layer's geometry");
    }
    if (k == Kind::Fp8) sh = Shared::Fp8Args;
    else if (k == Kind::Mxfp8) sh = Shared::Mxfp8Dense;
    else if (fp4 && d.shared[0].format == d.routed[0].format && d.shared_inter == d.cfg.inter) sh = Shared::Fp4Table;
    else refuse("an FP4 shared expert rides the routed experts' table: same format and width as they");
  } else if (d.cfg.n_shared_experts != 0) {
    refuse("n_shared_experts is set and no shared tensors are given");
  }
  auto cut_for = [&](int which, int64_t width) {   // gate / up: rows; down: columns
    return Cut{which == 2 ? 1 : 0, d.rank * width, width, whole};
  };
  const size_t n_globals = nvfp4 ? static_cast<size_t>(E + (sh == Shared::Fp4Table ? 1 : 0)) * 3 : 0;
  std::vector<DgppMoeExpertView> views(static_cast<size_t>(E + (sh == Shared::Fp4Table ? 1 : 0)) * 3);
  std::vector<float> globals(n_globals);
  DeviceMatrix shared_dev[3];
  const uint16_t* gate_dev = nullptr;
  const float* bias_dev = nullptr;
  for (int pass = 0; pass < 2; ++pass) {
    const bool dry = pass == 0;
    Bump bump;
    if (!dry) {
      bump.base = static_cast<uint8_t*>(out.arena);
      bump.cap = out.bytes;
    }
    float* globals_dev = reinterpret_cast<float*>(bump.take(n_globals * 4));
    for (int i = 0; i < E * 3; ++i) {
      const DeviceMatrix m = place(d.routed[i], cut_for(i % 3, M), bump, dry);
      if (dry) continue;
      if (fp4) {
        if (nvfp4) globals[static_cast<size_t>(i)] = nvfp4_divisor(d.routed[i]);
        DgppFp4Matrix f{m.payload, m.scales, nvfp4 ? globals_dev + i : nullptr, m.rows, m.cols, fp4_group_of(d.routed[i].format), 0, nullptr};
        loader_ok(dgpp_expert_view_from_fp4(&f, &views[static_cast<size_t>(i)]));
      } else {
        DgppQuantMatrix q{m.payload, reinterpret_cast<const float*>(m.scales), nullptr, m.rows, m.cols, m.block_rows, m.block_cols};
        loader_ok(dgpp_expert_view_from_quant(&q, &views[static_cast<size_t>(i)]));
      }
    }
    if (sh != Shared::None) {
      for (int i = 0; i < 3; ++i) {
        shared_dev[i] = place(d.shared[i], cut_for(i, SM), bump, dry);
        if (dry || sh != Shared::Fp4Table) continue;
        const size_t at = static_cast<size_t>(E) * 3 + i;
        if (nvfp4) globals[at] = nvfp4_divisor(d.shared[i]);
        DgppFp4Matrix f{shared_dev[i].payload, shared_dev[i].scales, nvfp4 ? globals_dev + at : nullptr, shared_dev[i].rows,
                        shared_dev[i].cols, fp4_group_of(d.shared[i].format), 0, nullptr};
        loader_ok(dgpp_expert_view_from_fp4(&f, &views[at]));
      }
    }
    uint8_t* gate_at = nullptr;
    uint8_t* bias_at = nullptr;
    if (d.router_weight) {
      if (d.router_weight->dtype != DGPP_DT_BF16 || d.router_weight->numel != static_cast<uint64_t>(E) * d.cfg.hidden)
        refuse("the router weight is BF16 [n_experts, hidden]");
      gate_at = bump.take(d.router_weight->nbytes);
    }
    if (d.router_bias) {
      if (d.router_bias->numel != static_cast<uint64_t>(E) || (d.router_bias->dtype != DGPP_DT_F32 && d.router_bias->dtype != DGPP_DT_BF16))
        refuse("the router bias is F32 or BF16 [n_experts]");
      bias_at = bump.take(static_cast<size_t>(E) * 4);
    }
    if (dry) {
      out.bytes = bump.used;
      hip_ok(hipMalloc(&out.arena, out.bytes ? out.bytes : 256), "hipMalloc");
      continue;
    }
    if (n_globals) to_device(reinterpret_cast<uint8_t*>(globals_dev), globals.data(), n_globals * 4);
    if (gate_at) {
      if (!d.router_weight->data) refuse("the router weight has no data");
      to_device(gate_at, d.router_weight->data, d.router_weight->nbytes);
      gate_dev = reinterpret_cast<const uint16_t*>(gate_at);
    }
    if (bias_at) {
      if (!d.router_bias->data) refuse("the router bias has no data");
      std::vector<float> b(static_cast<size_t>(E));
      if (d.router_bias->dtype == DGPP_DT_F32) {
        std::memcpy(b.data(), d.router_bias->data, b.size() * 4);
      } else {
        for (int e = 0; e < E; ++e) {
          uint16_t h;
          std::memcpy(&h, static_cast<const uint8_t*>(d.router_bias->data) + e * 2, 2);
          const uint32_t u = static_cast<uint32_t>(h) << 16;
          std::memcpy(&b[static_cast<size_t>(e)], &u, 4);
        }
      }
      to_device(bias_at, b.data(), b.size() * 4);
      bias_dev = reinterpret_cast<const float*>(bias_at);
    }
  }
  DgppMoeLayerDesc desc{};
  desc.cfg = d.cfg;
  desc.cfg.inter = static_cast<int32_t>(M);
  desc.expert_format = !fp4 ? DGPP_EXPERTS_FP8 : (nvfp4 ? DGPP_EXPERTS_NVFP4 : DGPP_EXPERTS_MXFP4);
  desc.max_tokens = d.max_tokens;
  desc.views = views.data();
  desc.shared_in_table = sh == Shared::Fp4Table ? 1 : 0;
  desc.shared_inter = sh == Shared::None ? 0 : static_cast<int32_t>(SM);
  desc.sh_rs = desc.sh_cs = 7;
  if (sh == Shared::Fp8Args) {
    // the slot kernels take ONE grid for the shared expert's three matrices
    for (int i = 1; i < 3; ++i)
      if (shared_dev[i].block_rows != shared_dev[0].block_rows || shared_dev[i].block_cols != shared_dev[0].block_cols)
        refuse("the shared expert's slices re-block to different scale grids (its width per rank must be a multiple of 128)");
    desc.sh_rs = shift_of(shared_dev[0].block_rows);
    desc.sh_cs = shift_of(shared_dev[0].block_cols);
    for (int i = 0; i < 3; ++i) {
      desc.sh_payload[i] = shared_dev[i].payload;
      desc.sh_scales[i] = reinterpret_cast<const float*>(shared_dev[i].scales);
    }
  } else if (sh == Shared::Mxfp8Dense) {
    for (int i = 0; i < 3; ++i) {
      desc.sh_payload[i] = shared_dev[i].payload;
      desc.sh_scales_e8m0[i] = shared_dev[i].scales;
    }
  }
  desc.router_gate = gate_dev;
  desc.router_bias = bias_dev;
  const int rc = dgpp_moe_layer_create(&desc, &out.layer);
  if (rc != DGPP_OK) throw Refused(rc, std::string("moe_resident_load: ") + dgpp_moe_layer_last_error());
  out.cfg = desc.cfg;
  out.shared_inter = desc.shared_inter;
}

}  // namespace

extern "C" {

const char* dgpp_moe_resident_last_error(void) { return g_resident_error.c_str(); }

int dgpp_moe_resident_load(const DgppMoeResidentDesc* desc, DgppMoeResident** out) {
  if (!desc || !out) {
    g_resident_error = "moe_resident_load: null argument";
    return DGPP_INVALID_ARGUMENT;
  }
  DgppMoeResident* r = new DgppMoeResident();
  try {
    load(*desc, *r);
    *out = r;
    return DGPP_OK;
  } catch (const Refused& e) {
    g_resident_error = e.what();
    dgpp_moe_resident_destroy(r);
    return e.code;
  } catch (const std::exception& e) {
    g_resident_error = e.what();
    dgpp_moe_resident_destroy(r);
    return DGPP_RUNTIME_ERROR;
  }
}

void dgpp_moe_resident_destroy(DgppMoeResident* r) {
  if (!r) return;
  if (r->layer) dgpp_moe_layer_destroy(r->layer);
  if (r->arena) (void)hipFree(r->arena);
  delete r;
}

DgppMoeLayer* dgpp_moe_resident_layer(DgppMoeResident* r) { return r ? r->layer : nullptr; }
size_t dgpp_moe_resident_weight_bytes(const DgppMoeResident* r) { return r ? r->bytes : 0; }
int dgpp_moe_resident_inter(const DgppMoeResident* r) { return r ? r->cfg.inter : 0; }

}  // extern "C"
