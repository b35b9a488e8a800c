// CPU oracle for the quantized MoE expert GEMV path — TEST INFRASTRUCTURE ONLY.
// See dgpp_oracle.h for the contract of every function and the reference lines it restates.
// Build: g++ -O2 -ffp-contract=off (no fused multiply-adds may be invented by the compiler:
// the fp32 accumulation chains below are bitwise contracts).
#include "dgpp_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

namespace {

inline uint32_t f2u(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
inline float u2f(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// The 8 e2m1 magnitudes, code order.
const float kE2m1Mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

// Positive e4m3 values by code 0..0x7E (0x7F is NaN), built once from the field definition.
struct E4m3Table {
  float v[127];
  E4m3Table() {
    for (int c = 0; c < 127; ++c) {
      const int e = c >> 3, m = c & 7;
      v[c] = e == 0 ? std::ldexp(static_cast<float>(m), -9)
                    : std::ldexp(1.0f + static_cast<float>(m) / 8.0f, e - 7);
    }
  }
};
const E4m3Table kE4m3;

// Nearest entry of an ascending table, ties to the even index.
template <int N>
int nearest_even(const float (&tab)[N], float a) {
  int hi = static_cast<int>(std::upper_bound(tab, tab + N, a) - tab);  // first > a
  if (hi == 0) return 0;
  if (hi == N) return N - 1;
  const int lo = hi - 1;
  const double dl = static_cast<double>(a) - tab[lo], dh = static_cast<double>(tab[hi]) - a;
  if (dl < dh) return lo;
  if (dh < dl) return hi;
  return (lo & 1) ? hi : lo;
}

inline double bf16d(uint16_t b) { return static_cast<double>(orc_bf16_to_f32(b)); }
inline uint16_t d2bf16(double v) { return orc_f32_to_bf16(static_cast<float>(v)); }

// An e8m0 byte as the fp8 dequant bridge reads it: the float whose exponent field is the byte.
inline float e8m0_as_bridge_float(uint8_t b) { return b ? u2f(static_cast<uint32_t>(b) << 23) : u2f(0x00400000u); }

// Runs fn(begin, end) over [0, n) on `threads` workers.
template <class Fn>
void parallel_rows(int64_t n, int threads, Fn fn) {
  if (threads <= 1 || n < 2) {
    fn(static_cast<int64_t>(0), n);
    return;
  }
  const int t = static_cast<int>(std::min<int64_t>(threads, n));
  std::vector<std::thread> pool;
  for (int i = 0; i < t; ++i) pool.emplace_back([=] { fn(n * i / t, n * (i + 1) / t); });
  for (auto& th : pool) th.join();
}

void dequant_matrix(const OrcMatrix& m, int64_t rows, int64_t cols, int threads, std::vector<double>& w) {
  w.resize(static_cast<size_t>(rows) * cols);
  parallel_rows(rows, threads, [&](int64_t r0, int64_t r1) {
    for (int64_t r = r0; r < r1; ++r) {
      double* o = w.data() + r * cols;
      if (m.kind == 0) {
        const int64_t sc = (cols + (1LL << m.cs) - 1) >> m.cs;
        for (int64_t c = 0; c < cols; ++c) {
          const float dec = orc_e4m3_to_f32(m.payload[r * cols + c]);
          const int64_t si = (r >> m.rs) * sc + (c >> m.cs);
          const float s = m.scales_f32 ? m.scales_f32[si] : e8m0_as_bridge_float(m.scales_u8[si]);
          o[c] = bf16d(orc_f32_to_bf16(dec * s));
        }
      } else {
        const int64_t pc = cols / 2, sc = cols / m.group;
        for (int64_t c = 0; c < cols; ++c) {
          const uint8_t byte = m.payload[r * pc + c / 2];
          const uint8_t code = (c & 1) ? byte >> 4 : byte & 0xF;
          const uint8_t sb = m.scales_u8[r * sc + c / m.group];
          const double s = m.group == 32 ? (sb == 255 ? std::nan("") : std::ldexp(1.0, static_cast<int>(sb) - 127))
                                         : static_cast<double>(orc_e4m3_to_f32(sb));
          o[c] = static_cast<double>(orc_e2m1_to_f32(code)) * s;
        }
      }
    }
  });
}

// out[n] = sum_k x[k] * w[n, k] / divisor, rows spread over threads.
void dots(const double* x, const std::vector<double>& w, int n, int k, double divisor, int threads, double* out) {
  parallel_rows(n, threads, [&](int64_t r0, int64_t r1) {
    for (int64_t r = r0; r < r1; ++r) {
      const double* wr = w.data() + r * k;
      double acc = 0.0;
      for (int kk = 0; kk < k; ++kk) acc += x[kk] * wr[kk];
      out[r] = acc / divisor;
    }
  });
}

double bf16_ulp(double x) {
  if (x == 0.0) return std::ldexp(1.0, -133);
  int e = 0;
  std::frexp(x, &e);
  return std::ldexp(1.0, e - 8);
}

template <class Got>
void compare_impl(const Got* got, const double* oracle, int64_t n, double ulp_budget, double floor_frac,
                  OrcCompare* rep, double (*widen)(Got)) {
  OrcCompare r{};
  r.total = n;
  double max_abs = 0;
  for (int64_t i = 0; i < n; ++i)
    if (!std::isnan(oracle[i])) max_abs = std::max(max_abs, std::fabs(oracle[i]));
  const double floor_abs = floor_frac * max_abs;
  double d2 = 0, o2 = 0;
  for (int64_t i = 0; i < n; ++i) {
    const double o = oracle[i], g = widen(got[i]);
    if (std::isnan(o) || std::isnan(g)) {
      if (std::isnan(o) != std::isnan(g)) {
        ++r.nan_pattern_errors;
        ++r.mismatches;
      }
      continue;
    }
    if (std::isinf(o) || std::isinf(g)) {
      if (o != g) ++r.mismatches;
      continue;
    }
    const double d = std::fabs(g - o);
    d2 += d * d;
    o2 += o * o;
    const double rel = d / std::max(std::fabs(o), floor_abs > 0 ? floor_abs : std::numeric_limits<double>::min());
    r.max_rel = std::max(r.max_rel, rel);
    if (d > floor_abs) r.max_ulps = std::max(r.max_ulps, d / bf16_ulp(o));
    if (d > ulp_budget * bf16_ulp(o) && d > floor_abs) ++r.mismatches;
  }
  r.l2_rel = o2 > 0 ? std::sqrt(d2 / o2) : 0.0;
  *rep = r;
}

}  // namespace

extern "C" {

float orc_bf16_to_f32(uint16_t bits) { return u2f(static_cast<uint32_t>(bits) << 16); }

uint16_t orc_f32_to_bf16(float v) {
  const uint32_t u = f2u(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u)  // NaN: canonical quiet NaN, sign kept
    return static_cast<uint16_t>(((u >> 16) & 0x8000u) | 0x7FC0u);
  const uint32_t keep_odd = (u >> 16) & 1u;
  return static_cast<uint16_t>((u + 0x7FFFu + keep_odd) >> 16);
}

float orc_e4m3_to_f32(uint8_t code) {
  const uint32_t sign = static_cast<uint32_t>(code & 0x80u) << 24;
  const int c = code & 0x7F;
  if (c == 0x7F) return u2f(0x7FC00000u | sign);
  return u2f(f2u(kE4m3.v[c]) | sign);
}

uint8_t orc_f32_to_e4m3(float v) {
  const uint32_t u = f2u(v);
  const uint8_t sign = static_cast<uint8_t>((u >> 24) & 0x80u);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return sign | 0x7F;
  float a = u2f(u & 0x7FFFFFFFu);
  if (a > 448.0f) a = 448.0f;  // saturating: nothing reaches the NaN code
  return sign | static_cast<uint8_t>(nearest_even(kE4m3.v, a));
}

float orc_e2m1_to_f32(uint8_t code) {
  const float mag = kE2m1Mag[code & 7];
  return (code & 8) ? -mag : mag;
}

uint8_t orc_f32_to_e2m1(float v) {
  const uint32_t u = f2u(v);
  const uint8_t sign = static_cast<uint8_t>((u >> 28) & 8u);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return sign | 7;  // no NaN code: saturate
  const float a = u2f(u & 0x7FFFFFFFu);
  return sign | static_cast<uint8_t>(nearest_even(kE2m1Mag, a));
}

float orc_e8m0_to_f32(uint8_t code) {
  if (code == 255) return u2f(0x7FC00000u);
  return static_cast<float>(std::ldexp(1.0, static_cast<int>(code) - 127));  // 2^-127 is an fp32 subnormal
}

uint8_t orc_e8m0_ceil_log2(float v) {
  // ceil(log2 v) from the IEEE fields: the exponent, plus one when the mantissa is not zero.
  const uint32_t u = f2u(v);
  const int field = static_cast<int>((u >> 23) & 0xFF);
  const int b = field + ((u & 0x7FFFFFu) ? 1 : 0);  // (field - 127 + carry) + 127
  return static_cast<uint8_t>(std::min(b, 254));
}

void orc_dequant_fp8(const uint8_t* payload, const float* scales_f32, const uint8_t* scales_e8m0,
                     int64_t rows, int64_t cols, int rs, int cs, int strict, double* out) {
  const int64_t sc = (cols + (1LL << cs) - 1) >> cs;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      const float dec = orc_e4m3_to_f32(payload[r * cols + c]);
      const int64_t si = (r >> rs) * sc + (c >> cs);
      const float s = scales_f32 ? scales_f32[si] : e8m0_as_bridge_float(scales_e8m0[si]);
      out[r * cols + c] = strict ? bf16d(orc_f32_to_bf16(dec * s)) : static_cast<double>(dec) * static_cast<double>(s);
    }
}

void orc_dequant_fp4(const uint8_t* payload, const uint8_t* scales, int group, int64_t rows,
                     int64_t cols, double* out) {
  OrcMatrix m{};
  m.payload = payload;
  m.scales_u8 = scales;
  m.kind = 1;
  m.group = group;
  std::vector<double> w;
  dequant_matrix(m, rows, cols, 1, w);
  std::memcpy(out, w.data(), w.size() * sizeof(double));
}

void orc_gemv_fp8(const uint16_t* act, int64_t act_stride, const uint8_t* payload,
                  const float* scales_f32, const uint8_t* scales_e8m0, int m, int n, int k, int rs,
                  int cs, int strict, double* out_raw) {
  std::vector<double> w(static_cast<size_t>(n) * std::max(k, 1));
  if (k > 0) orc_dequant_fp8(payload, scales_f32, scales_e8m0, n, k, rs, cs, strict, w.data());
  for (int mm = 0; mm < m; ++mm)
    for (int nn = 0; nn < n; ++nn) {
      double acc = 0.0;
      for (int kk = 0; kk < k; ++kk) acc += bf16d(act[mm * act_stride + kk]) * w[static_cast<size_t>(nn) * k + kk];
      out_raw[static_cast<size_t>(mm) * n + nn] = acc;
    }
}

void orc_gemv_fp4(const uint16_t* act, int64_t act_stride, const uint8_t* payload,
                  const uint8_t* scales, double divisor, int group, int m, int n, int k,
                  double* out_raw) {
  std::vector<double> w(static_cast<size_t>(n) * k);
  orc_dequant_fp4(payload, scales, group, n, k, w.data());
  for (int mm = 0; mm < m; ++mm)
    for (int nn = 0; nn < n; ++nn) {
      double acc = 0.0;
      for (int kk = 0; kk < k; ++kk) acc += bf16d(act[mm * act_stride + kk]) * w[static_cast<size_t>(nn) * k + kk];
      out_raw[static_cast<size_t>(mm) * n + nn] = acc / divisor;
    }
}

void orc_router_scores(const uint16_t* hidden, const uint16_t* gate, const float* bias, int mode,
                       int tokens, int experts, int hidden_dim, double* scores, double* biased) {
  for (int t = 0; t < tokens; ++t)
    for (int e = 0; e < experts; ++e) {
      double dot = 0.0;
      for (int k = 0; k < hidden_dim; ++k)
        dot += bf16d(hidden[static_cast<size_t>(t) * hidden_dim + k]) * bf16d(gate[static_cast<size_t>(e) * hidden_dim + k]);
      double s, b;
      if (mode == ORC_ROUTER_SOFTMAX) {
        s = bf16d(d2bf16(dot));
        b = s;
      } else if (mode == ORC_ROUTER_SQRT_SOFTPLUS) {
        s = std::sqrt(dot > 20.0 ? dot : std::log1p(std::exp(dot)));
        b = s + bias[e];
      } else {
        s = 1.0 / (1.0 + std::exp(-dot));
        b = s + bias[e];
      }
      scores[static_cast<size_t>(t) * experts + e] = s;
      biased[static_cast<size_t>(t) * experts + e] = b;
    }
}

void orc_router_select(const double* scores, const double* biased, int mode, int tokens,
                       int experts, int top_k, double scaling, int norm_topk, int32_t* ids,
                       float* weights) {
  std::vector<double> p(experts);
  std::vector<char> used(experts);
  std::vector<std::pair<int, double>> picks(top_k);
  for (int t = 0; t < tokens; ++t) {
    const double* srow = scores + static_cast<size_t>(t) * experts;
    const double* brow = biased + static_cast<size_t>(t) * experts;
    if (mode == ORC_ROUTER_SOFTMAX) {
      double mx = -INFINITY, sum = 0.0;
      for (int e = 0; e < experts; ++e) mx = std::max(mx, srow[e]);
      for (int e = 0; e < experts; ++e) sum += std::exp(srow[e] - mx);
      for (int e = 0; e < experts; ++e) p[e] = std::exp(srow[e] - mx) / sum;
    } else {
      for (int e = 0; e < experts; ++e) p[e] = srow[e];
    }
    std::fill(used.begin(), used.end(), 0);
    for (int r = 0; r < top_k; ++r) {
      int best = -1;
      double bv = -INFINITY;
      for (int e = 0; e < experts; ++e)
        if (!used[e] && brow[e] > bv) {
          bv = brow[e];
          best = e;
        }
      if (best < 0) {  // every remaining key is -inf or NaN: the first unused id (never in the tests)
        for (int e = 0; e < experts && best < 0; ++e)
          if (!used[e]) best = e;
      }
      used[best] = 1;
      picks[r] = {best, p[best]};
    }
    std::stable_sort(picks.begin(), picks.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    double denom = 0.0;
    for (int r = 0; r < top_k; ++r) denom += picks[r].second;
    denom += 1e-20;
    for (int r = 0; r < top_k; ++r) {
      double w = norm_topk ? (picks[r].second / denom) * scaling : picks[r].second * scaling;
      if (mode == ORC_ROUTER_SOFTMAX) w = bf16d(d2bf16(w));
      ids[static_cast<size_t>(t) * top_k + r] = picks[r].first;
      weights[static_cast<size_t>(t) * top_k + r] = static_cast<float>(w);
    }
  }
}

void orc_moe_segment(const int32_t* ids, int tokens, int top_k, int experts, int32_t* rows,
                     int32_t* slot_row, int32_t* segs) {
  const int tk = tokens * top_k;
  std::vector<int> count(experts, 0), next(experts, 0);
  for (int i = 0; i < tk; ++i) ++count[ids[i]];
  int acc = 0;
  for (int e = 0; e < experts; ++e) {
    segs[e * 3 + 0] = acc;
    segs[e * 3 + 1] = count[e];
    segs[e * 3 + 2] = e;
    next[e] = acc;
    acc += count[e];
  }
  for (int i = 0; i < tk; ++i) {  // (token, slot) order => stable inside an expert
    const int pos = next[ids[i]]++;
    rows[pos] = i / top_k;
    slot_row[i] = pos;
  }
  segs[experts * 3 + 0] = tk;
  segs[experts * 3 + 1] = tokens;
  segs[experts * 3 + 2] = experts;
  for (int t = 0; t < tokens; ++t) rows[tk + t] = t;
}

void orc_moe_slot_order(const int32_t* ids, int slots, int top_k, int experts, int shared_early,
                        int32_t* order, int32_t* runs) {
  std::vector<int> key(slots), sorted(slots);
  for (int s = 0; s < slots; ++s) {
    const int t = s / (top_k + 1), j = s % (top_k + 1);
    key[s] = j < top_k ? ids[t * top_k + j] : experts;
  }
  const int tokens = slots / (top_k + 1), routed = tokens * top_k;
  for (int s = 0; s < slots; ++s) {
    int pos = 0;
    for (int o = 0; o < slots; ++o) pos += (key[o] < key[s]) || (key[o] == key[s] && o < s);
    if (shared_early) pos = pos < routed ? pos + std::min(pos, tokens) : 2 * (pos - routed) + 1;
    order[pos] = s;
    sorted[pos] = key[s];
  }
  if (!runs) return;
  const int group_rows = 64, tile_rows = 16;
  int32_t* list = runs + slots;
  int n_list = 0;
  for (int p = 0; p < slots; ++p) {
    int len = 0;
    if (p == 0 || sorted[p - 1] != sorted[p]) {
      len = 1;
      while (p + len < slots && sorted[p + len] == sorted[p]) ++len;
    }
    runs[p] = len;
    if (len > tile_rows)
      for (int r0 = 0; r0 < len; r0 += group_rows) list[n_list++] = (p + r0) | (std::min(group_rows, len - r0) << 16);
  }
  for (int i = n_list; i < slots / (tile_rows + 1) + 1; ++i) list[i] = -1;
}

int orc_moe_tile_list(const int32_t* segs, int n_segs, int tile_rows, int32_t* tiles) {
  int n = 0;
  for (int s = 0; s < n_segs; ++s)
    for (int m0 = 0; m0 < segs[s * 3 + 1]; m0 += tile_rows) {
      tiles[n * 2 + 0] = s;
      tiles[n * 2 + 1] = m0;
      ++n;
    }
  return n;
}

void orc_compact_segments(const int32_t* segs_in, int32_t* segs_out, int experts, int capacity) {
  int at = 0;
  for (int e = 0; e < experts; ++e)
    if (segs_in[e * 3 + 1] > 0) {
      if (at < capacity) std::memcpy(segs_out + at * 3, segs_in + e * 3, 12);
      ++at;
    }
  for (int i = at; i < capacity; ++i) segs_out[i * 3] = segs_out[i * 3 + 1] = segs_out[i * 3 + 2] = 0;
}

void orc_swiglu(const uint16_t* gate, const uint16_t* up, int64_t n, float limit, uint16_t* out) {
  const double lim = static_cast<double>(limit);
  for (int64_t i = 0; i < n; ++i) {
    double g = bf16d(gate[i]), u = bf16d(up[i]);
    if (g > lim) g = lim;
    u = std::min(std::max(u, -lim), lim);
    const uint16_t silu = d2bf16(g * (1.0 / (1.0 + std::exp(-g))));
    out[i] = d2bf16(bf16d(silu) * u);
  }
}

void orc_slot_accum(const float* contrib, const float* weights, int tokens, int hidden, int top_k,
                    int with_shared, float* out_f32, uint16_t* out_bf16) {
  for (int t = 0; t < tokens; ++t)
    for (int c = 0; c < hidden; ++c) {
      const size_t base = static_cast<size_t>(t) * (top_k + 1);
      float a = 0.f;
      for (int j = 0; j < top_k; ++j)
        a = std::fmaf(weights[static_cast<size_t>(t) * top_k + j], contrib[(base + j) * hidden + c], a);
      if (with_shared) a = std::fmaf(1.0f, contrib[(base + top_k) * hidden + c], a);
      if (out_f32) out_f32[static_cast<size_t>(t) * hidden + c] = a;
      if (out_bf16) out_bf16[static_cast<size_t>(t) * hidden + c] = orc_f32_to_bf16(a);
    }
}

void orc_accum_ordered(const float* down, int64_t down_stride, const int32_t* slot_row,
                       const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                       int top_k, int hidden, float* out_f32, uint16_t* out_bf16) {
  std::vector<int> ord(top_k);
  for (int t = 0; t < tokens; ++t) {
    for (int j = 0; j < top_k; ++j) ord[j] = j;
    std::stable_sort(ord.begin(), ord.end(),
                     [&](int a, int b) { return slot_ids[t * top_k + a] < slot_ids[t * top_k + b]; });
    for (int h = 0; h < hidden; ++h) {
      float a = 0.f;
      for (int j = 0; j < top_k; ++j) {
        const int s = t * top_k + ord[j];
        a = std::fmaf(slot_w[s], down[static_cast<size_t>(slot_row[s]) * down_stride + h], a);
      }
      if (shared_row0 >= 0) a = std::fmaf(1.0f, down[static_cast<size_t>(shared_row0 + t) * down_stride + h], a);
      if (out_f32) out_f32[static_cast<size_t>(t) * hidden + h] = a;
      if (out_bf16) out_bf16[static_cast<size_t>(t) * hidden + h] = orc_f32_to_bf16(a);
    }
  }
}

void orc_moe_forward(const uint16_t* x, int64_t x_stride, const int32_t* ids, const float* weights,
                     int tokens, int top_k, int hidden, int inter, int shared_inter,
                     const OrcMatrix* experts, const OrcMatrix* shared, float swiglu_limit,
                     int threads, double* out_raw, uint16_t* out_bf16) {
  std::vector<double> wg, wu, wd, xd(hidden), actd, gate, up, down(hidden), acc(hidden);
  std::vector<uint16_t> gb, ub, act;
  auto expert_pass = [&](const OrcMatrix* m3, int I, double weight) {
    dequant_matrix(m3[0], I, hidden, threads, wg);
    dequant_matrix(m3[1], I, hidden, threads, wu);
    dequant_matrix(m3[2], hidden, I, threads, wd);
    gate.resize(I);
    up.resize(I);
    gb.resize(I);
    ub.resize(I);
    act.resize(I);
    actd.resize(I);
    dots(xd.data(), wg, I, hidden, m3[0].divisor, threads, gate.data());
    dots(xd.data(), wu, I, hidden, m3[1].divisor, threads, up.data());
    for (int i = 0; i < I; ++i) {
      gb[i] = d2bf16(gate[i]);
      ub[i] = d2bf16(up[i]);
    }
    orc_swiglu(gb.data(), ub.data(), I, swiglu_limit, act.data());
    for (int i = 0; i < I; ++i) actd[i] = bf16d(act[i]);
    dots(actd.data(), wd, hidden, I, m3[2].divisor, threads, down.data());
    for (int d = 0; d < hidden; ++d) acc[d] += weight * down[d];
  };
  for (int t = 0; t < tokens; ++t) {
    for (int k = 0; k < hidden; ++k) xd[k] = bf16d(x[static_cast<size_t>(t) * x_stride + k]);
    std::fill(acc.begin(), acc.end(), 0.0);
    for (int j = 0; j < top_k; ++j) {
      const int e = ids[static_cast<size_t>(t) * top_k + j];
      expert_pass(experts + static_cast<size_t>(e) * 3, inter, static_cast<double>(weights[static_cast<size_t>(t) * top_k + j]));
    }
    if (shared) expert_pass(shared, shared_inter, 1.0);
    for (int d = 0; d < hidden; ++d) {
      if (out_raw) out_raw[static_cast<size_t>(t) * hidden + d] = acc[d];
      if (out_bf16) out_bf16[static_cast<size_t>(t) * hidden + d] = d2bf16(acc[d]);
    }
  }
}

void orc_shared_gate(const uint16_t* x, int64_t x_stride, const uint16_t* g, int tokens, int hidden, float* w) {
  for (int t = 0; t < tokens; ++t) {
    if (!g) {
      w[t] = 1.0f;
      continue;
    }
    double logit = 0.0;
    for (int k = 0; k < hidden; ++k) logit += bf16d(x[static_cast<size_t>(t) * x_stride + k]) * bf16d(g[k]);
    logit = bf16d(d2bf16(logit));
    w[t] = static_cast<float>(bf16d(d2bf16(1.0 / (1.0 + std::exp(-logit)))));
  }
}

// src/kernels/glm_moe.cu:917-949: routes from a table; the weights' chain in fp32 (fadd from zero in row order, + 1e-20,
// one division and one multiplication per weight - this file is compiled with -ffp-contract=off).
void orc_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int n_tokens, int vocab,
                     int n_experts, int top_k, float scaling, int norm_topk, int32_t* ids, float* weights) {
  for (int t = 0; t < n_tokens; ++t) {
    int64_t tok = tokens[t];
    if (tok < 0 || tok >= vocab) tok = 0;
    const int32_t* row = tid2eid + tok * top_k;
    float denom = 0.f;
    for (int i = 0; i < top_k; ++i) denom = denom + scores[static_cast<size_t>(t) * n_experts + row[i]];
    denom = denom + 1e-20f;
    for (int i = 0; i < top_k; ++i) {
      const float v = scores[static_cast<size_t>(t) * n_experts + row[i]];
      ids[static_cast<size_t>(t) * top_k + i] = row[i];
      weights[static_cast<size_t>(t) * top_k + i] = norm_topk ? (v / denom) * scaling : v * scaling;
    }
  }
}

// ---- activation-quantized NVFP4 form -----------------------------------------------------------
// src/kernels/moe_w4a4.cu:139-236: per row a global, per 16 elements an e4m3 scale, e2m1 codes. Plain fp32 operations
// in the reference's order (this file is compiled with -ffp-contract=off).
void orc_nvfp4_quantize_rows(const uint16_t* x, int64_t stride, int rows, int k, float static_gs, uint8_t* codes,
                             uint8_t* scales, int64_t scale_stride, float* gs) {
  const int groups = k / 16;
  for (int r = 0; r < rows; ++r) {
    const uint16_t* src = x + static_cast<size_t>(r) * stride;
    float row_amax = 0.f;
    for (int c = 0; c < k; ++c) row_amax = std::max(row_amax, std::fabs(orc_bf16_to_f32(src[c])));
    const float global = static_gs > 0.f ? static_gs : (row_amax > 0.f ? row_amax / (6.f * 448.f) : 1.f);
    gs[r] = global;
    for (int g = 0; g < groups; ++g) {
      float gmax = 0.f;
      for (int i = 0; i < 16; ++i) gmax = std::max(gmax, std::fabs(orc_bf16_to_f32(src[g * 16 + i])));
      uint8_t* code = codes + static_cast<size_t>(r) * (k / 2) + static_cast<size_t>(g) * 8;
      const uint8_t sb = orc_f32_to_e4m3(gmax / (6.f * global));
      const float bs = orc_e4m3_to_f32(sb);
      if (gmax == 0.f || bs == 0.f) {
        scales[static_cast<size_t>(r) * scale_stride + g] = 0;
        for (int i = 0; i < 8; ++i) code[i] = 0;
        continue;
      }
      scales[static_cast<size_t>(r) * scale_stride + g] = sb;
      const float q = 1.f / (bs * global);
      for (int i = 0; i < 8; ++i) {
        const uint8_t lo = orc_f32_to_e2m1(orc_bf16_to_f32(src[g * 16 + 2 * i]) * q);
        const uint8_t hi = orc_f32_to_e2m1(orc_bf16_to_f32(src[g * 16 + 2 * i + 1]) * q);
        code[i] = static_cast<uint8_t>(lo | (hi << 4));
      }
    }
  }
}

// src/kernels/minimax_native_moe.cu:36-85 with every reciprocal correctly rounded (the reference's is NVIDIA's
// approximate instruction): decode = amax * (1 / 2688), encode = 1 / decode (FLT_MAX for a zero row),
// scale = e4m3(encode * (amax16 * (1 / 6))), inverse = 1 / (float(scale) * (1 / encode)) (0 for a zero scale).
void orc_minimax_quantize_rows_nvfp4(const uint16_t* x, int64_t stride, int rows, int k, uint8_t* codes, uint8_t* scales,
                                     float* globals) {
  const int groups = k / 16;
  for (int r = 0; r < rows; ++r) {
    const uint16_t* src = x + static_cast<size_t>(r) * stride;
    float row_max = 0.f;
    for (int c = 0; c < k; ++c) row_max = std::max(row_max, std::fabs(orc_bf16_to_f32(src[c])));
    const float decode = row_max * (1.f / (6.f * 448.f));
    const float encode = row_max == 0.f ? std::numeric_limits<float>::max() : 1.f / decode;
    globals[r] = decode;
    for (int g = 0; g < groups; ++g) {
      float gmax = 0.f;
      for (int i = 0; i < 16; ++i) gmax = std::max(gmax, std::fabs(orc_bf16_to_f32(src[g * 16 + i])));
      const float sixth = 1.f / 6.f;
      const float scaled_max = gmax * sixth;
      const uint8_t sb = orc_f32_to_e4m3(encode * scaled_max);
      const float sv = orc_e4m3_to_f32(sb);
      const float back = 1.f / encode;
      const float inverse = sv == 0.f ? 0.f : 1.f / (sv * back);
      scales[static_cast<size_t>(r) * groups + g] = sb;
      uint8_t* code = codes + static_cast<size_t>(r) * (k / 2) + static_cast<size_t>(g) * 8;
      for (int i = 0; i < 8; ++i) {
        const uint8_t lo = orc_f32_to_e2m1(orc_bf16_to_f32(src[g * 16 + 2 * i]) * inverse);
        const uint8_t hi = orc_f32_to_e2m1(orc_bf16_to_f32(src[g * 16 + 2 * i + 1]) * inverse);
        code[i] = static_cast<uint8_t>(lo | (hi << 4));
      }
    }
  }
}

// src/kernels/minimax_native_moe.cu:87-95 in double, rounded once to BF16 (the kernel evaluates it in fp32).
void orc_minimax_swiglu_f32(const float* gate, const float* up, int64_t count, double alpha, double limit, uint16_t* out,
                            double* out_exact) {
  for (int64_t i = 0; i < count; ++i) {
    const double g = std::min(static_cast<double>(gate[i]), limit);
    const double u = std::min(std::max(static_cast<double>(up[i]), -limit), limit);
    const double v = (g / (1.0 + std::exp(-alpha * g))) * (u + 1.0);
    if (out) out[i] = d2bf16(v);
    if (out_exact) out_exact[i] = v;
  }
}

// The MiniMax router as its CPU statement does it (src/models/minimax/reference.cpp:96-113) and its kernels
// (src/kernels/minimax.cu:409-440), in FP32 throughout: ranking by score + bias (ties to the lower id), ids
// ascending, weights = score / max(sum in id order, 1e-20) * factor. `scores` are the sigmoid scores themselves
// (the device's, when a device selection is checked against this).
void orc_minimax_route_scores(const float* scores, const float* bias, int rows, int experts, int topk, float factor,
                              int32_t* ids, float* weights) {
  std::vector<int> order(static_cast<size_t>(experts));
  for (int r = 0; r < rows; ++r) {
    const float* row = scores + static_cast<size_t>(r) * experts;
    for (int e = 0; e < experts; ++e) order[static_cast<size_t>(e)] = e;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
      const float sa = row[a] + bias[a], sb = row[b] + bias[b];
      return sa == sb ? a < b : sa > sb;
    });
    std::vector<int> picked(order.begin(), order.begin() + topk);
    std::sort(picked.begin(), picked.end());
    float sum = 0.f;
    for (int e : picked) sum += row[e];
    for (int j = 0; j < topk; ++j) {
      ids[static_cast<size_t>(r) * topk + j] = picked[static_cast<size_t>(j)];
      weights[static_cast<size_t>(r) * topk + j] = row[picked[static_cast<size_t>(j)]] / std::max(sum, 1e-20f) * factor;
    }
  }
}
// scores[r, e] = sigmoid(dot(x[r], gate[e])) with the dot in double (x BF16 bits, gate FP32): what the device's FP32
// chain is held against. src/kernels/minimax.cu:397-408
void orc_minimax_router_scores(const uint16_t* x, const float* gate, int rows, int hidden, int experts, double* scores) {
  for (int r = 0; r < rows; ++r)
    for (int e = 0; e < experts; ++e) {
      double dot = 0.0;
      for (int k = 0; k < hidden; ++k)
        dot += bf16d(x[static_cast<size_t>(r) * hidden + k]) *
               static_cast<double>(gate[static_cast<size_t>(e) * hidden + k]);
      scores[static_cast<size_t>(r) * experts + e] = 1.0 / (1.0 + std::exp(-dot));
    }
}

void orc_w4a4_gemm(const uint8_t* a_codes, const uint8_t* a_scales, int64_t a_scale_stride, const float* a_gs,
                   const uint8_t* w_codes, const uint8_t* w_scales, double w_global, int m, int n, int k, double* out,
                   double* out_abs) {
  std::vector<double> a(static_cast<size_t>(m) * k), w(static_cast<size_t>(n) * k);
  for (int r = 0; r < m; ++r)
    for (int c = 0; c < k; ++c) {
      const uint8_t b = a_codes[static_cast<size_t>(r) * (k / 2) + c / 2];
      a[static_cast<size_t>(r) * k + c] = static_cast<double>(orc_e2m1_to_f32(c % 2 ? b >> 4 : b & 15)) *
                                          static_cast<double>(orc_e4m3_to_f32(a_scales[static_cast<size_t>(r) * a_scale_stride + c / 16])) *
                                          static_cast<double>(a_gs[r]);
    }
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < k; ++c) {
      const uint8_t b = w_codes[static_cast<size_t>(r) * (k / 2) + c / 2];
      w[static_cast<size_t>(r) * k + c] = static_cast<double>(orc_e2m1_to_f32(c % 2 ? b >> 4 : b & 15)) *
                                          static_cast<double>(orc_e4m3_to_f32(w_scales[static_cast<size_t>(r) * (k / 16) + c / 16])) /
                                          w_global;
    }
  for (int r = 0; r < m; ++r)
    for (int c = 0; c < n; ++c) {
      double dot = 0.0, mag = 0.0;
      for (int kk = 0; kk < k; ++kk) {
        const double t = a[static_cast<size_t>(r) * k + kk] * w[static_cast<size_t>(c) * k + kk];
        dot += t;
        mag += std::fabs(t);
      }
      out[static_cast<size_t>(r) * n + c] = dot;
      if (out_abs) out_abs[static_cast<size_t>(r) * n + c] = mag;
    }
}

// ---- activation-quantized MXFP8 form ---------------------------------------------------------

void orc_mxfp8_quantize_rows(const uint16_t* x, int64_t stride, int rows, int k, uint8_t* codes, uint8_t* scales) {
  const int groups = k / 32;
  for (int r = 0; r < rows; ++r)
    for (int g = 0; g < groups; ++g) {
      const uint16_t* src = x + static_cast<size_t>(r) * stride + static_cast<size_t>(g) * 32;
      float maximum = 0.f;
      for (int i = 0; i < 32; ++i) maximum = std::max(maximum, std::fabs(orc_bf16_to_f32(src[i])));
      // ceil(log2(maximum / 448)) off the float's fields: 448 = 1.75 * 2^8, so the ceiling is the
      // exponent less 8, plus one when the significand exceeds 1.75.
      const uint32_t u = f2u(maximum);
      const int field = static_cast<int>((u >> 23) & 0xFF);
      const int exponent = std::max(-127, field - 127 - 8 + ((u & 0x7FFFFFu) > 0x600000u ? 1 : 0));
      // 2^-exponent is a float for every exponent the rule can produce (-127 .. 120).
      const float inverse = static_cast<float>(std::ldexp(1.0, -exponent));
      for (int i = 0; i < 32; ++i)
        codes[static_cast<size_t>(r) * k + static_cast<size_t>(g) * 32 + i] = orc_f32_to_e4m3(orc_bf16_to_f32(src[i]) * inverse);
      scales[static_cast<size_t>(r) * groups + g] = static_cast<uint8_t>(exponent + 127);
    }
}

void orc_swiglu_oai(const uint16_t* gate, const uint16_t* up, int64_t stride, int rows, int k, float alpha, float limit,
                    double* exact, uint16_t* rounded) {
  for (int r = 0; r < rows; ++r)
    for (int c = 0; c < k; ++c) {
      const size_t at = static_cast<size_t>(r) * stride + c, to = static_cast<size_t>(r) * k + c;
      const double g = std::min(bf16d(gate[at]), static_cast<double>(limit));
      const double u = std::min(std::max(bf16d(up[at]), -static_cast<double>(limit)), static_cast<double>(limit));
      const double v = g / (1.0 + std::exp(-static_cast<double>(alpha) * g)) * (u + 1.0);
      if (exact) exact[to] = v;
      if (rounded) rounded[to] = d2bf16(v);
    }
}

void orc_mxfp8_gemm(const uint8_t* a, const uint8_t* a_scales, const uint8_t* w, const uint8_t* w_scales, int m, int n, int k,
                    double* out, double* out_abs) {
  const int groups = k / 32;
  std::vector<double> ad(static_cast<size_t>(m) * k), wd(static_cast<size_t>(n) * k);
  for (int r = 0; r < m; ++r)
    for (int c = 0; c < k; ++c)
      ad[static_cast<size_t>(r) * k + c] = std::ldexp(static_cast<double>(orc_e4m3_to_f32(a[static_cast<size_t>(r) * k + c])),
                                                       static_cast<int>(a_scales[static_cast<size_t>(r) * groups + c / 32]) - 127);
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < k; ++c)
      wd[static_cast<size_t>(r) * k + c] = std::ldexp(static_cast<double>(orc_e4m3_to_f32(w[static_cast<size_t>(r) * k + c])),
                                                       static_cast<int>(w_scales[static_cast<size_t>(r) * groups + c / 32]) - 127);
  for (int r = 0; r < m; ++r)
    for (int c = 0; c < n; ++c) {
      double sum = 0, abs_sum = 0;
      const double* ar = &ad[static_cast<size_t>(r) * k];
      const double* wr = &wd[static_cast<size_t>(c) * k];
      for (int i = 0; i < k; ++i) {
        const double prod = ar[i] * wr[i];
        sum += prod;
        abs_sum += std::fabs(prod);
      }
      out[static_cast<size_t>(r) * n + c] = sum;
      if (out_abs) out_abs[static_cast<size_t>(r) * n + c] = abs_sum;
    }
}

void orc_compare_bf16(const uint16_t* got, const double* oracle, int64_t n, double ulp_budget,
                      double floor_frac, OrcCompare* rep) {
  compare_impl<uint16_t>(got, oracle, n, ulp_budget, floor_frac, rep, [](uint16_t b) { return bf16d(b); });
}

void orc_compare_f32(const float* got, const double* oracle, int64_t n, double ulp_budget,
                     double floor_frac, OrcCompare* rep) {
  compare_impl<float>(got, oracle, n, ulp_budget, floor_frac, rep, [](float f) { return static_cast<double>(f); });
}

}  // extern "C"
