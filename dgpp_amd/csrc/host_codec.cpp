// Host-side pieces of the library: scalar codecs, the published weight-quantisation recipes and
// the seeded synthetic-data generators. Pure CPU code (compiled with -ffp-contract=off so the
// encoders' arithmetic is exactly the written operations).
//
// Recipes: block FP8 — src/loaders/fp8_quant.hpp:32-46; NVFP4 — src/loaders/nvfp4_quant.hpp:25-55;
// MXFP4 / MXFP8 — one E8M0 byte per 32 elements picked by the ceil-log2 rule of the reference's own
// E8M0 producers (src/kernels/latent_format.hpp:117-123, src/kernels/mxfp8_gemm.cu:61-66).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <thread>
#include <vector>

#include "../../include/dgpp_amd.h"
#include "numerics.hpp"

using namespace dgpp_amd;

namespace {

template <class Fn>
void parallel_for(int64_t n, int threads, Fn fn) {
  if (threads <= 0) threads = static_cast<int>(std::max(1u, std::min(16u, std::thread::hardware_concurrency())));
  if (threads == 1 || n < 2) {
    fn(static_cast<int64_t>(0), n);
    return;
  }
  const int t = static_cast<int>(std::min<int64_t>(threads, n));
  std::vector<std::thread> pool;
  for (int i = 0; i < t; ++i) pool.emplace_back([=] { fn(n * i / t, n * (i + 1) / t); });
  for (auto& th : pool) th.join();
}

struct XorShift64 {
  uint64_t s;
  explicit XorShift64(uint64_t seed) : s(seed | 1ull) {}
  uint64_t next() {
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return s;
  }
  double unit_open() { return (static_cast<double>(next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }  // (0, 1)
};

// A well-mixed per-block seed (splitmix64 finaliser) so blocks are independent streams.
uint64_t block_seed(uint64_t seed, uint64_t block) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * (block + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

constexpr int64_t kGenBlock = 4096;

template <class Store>
void fill_normal(uint64_t seed, float mean, float stddev, int64_t n, int threads, Store store) {
  const int64_t blocks = (n + kGenBlock - 1) / kGenBlock;
  parallel_for(blocks, threads, [&](int64_t b0, int64_t b1) {
    for (int64_t b = b0; b < b1; ++b) {
      XorShift64 rng(block_seed(seed, static_cast<uint64_t>(b)));
      for (int w = 0; w < 8; ++w) rng.next();
      const int64_t lo = b * kGenBlock, hi = std::min(n, lo + kGenBlock);
      for (int64_t i = lo; i < hi; i += 2) {
        const double u1 = rng.unit_open(), u2 = rng.unit_open();
        const double r = std::sqrt(-2.0 * std::log(u1));
        const double a = 6.283185307179586476925 * u2;
        store(i, static_cast<float>(mean + stddev * r * std::cos(a)));
        if (i + 1 < hi) store(i + 1, static_cast<float>(mean + stddev * r * std::sin(a)));
      }
    }
  });
}

// One E8M0-scaled block of 32: byte b = 127 + ceil(log2(amax / fmt_max)), scale 2^(b-127).
template <class Encode>
void encode_mx_rows(const float* src, int64_t rows, int64_t cols, float fmt_max, uint8_t* scales, int threads,
                    Encode encode_block) {
  const int64_t blocks_per_row = cols / 32;
  parallel_for(rows, threads, [&](int64_t r0, int64_t r1) {
    for (int64_t r = r0; r < r1; ++r)
      for (int64_t b = 0; b < blocks_per_row; ++b) {
        const float* v = src + r * cols + b * 32;
        float amax = 0.f;
        for (int j = 0; j < 32; ++j) amax = std::max(amax, std::fabs(v[j]));
        uint8_t byte = 0;
        float inv = 0.f;
        if (amax > 0.f && std::isfinite(amax)) {
          byte = e8m0_ceil_log2(amax / fmt_max);
          const float s = e8m0_to_f32(byte);
          inv = 1.0f / s;  // a power of two: exact
        }
        scales[r * blocks_per_row + b] = byte;
        encode_block(r, b, v, inv);
      }
  });
}

}  // namespace

extern "C" {

float dgpp_bf16_to_f32(uint16_t bits) { return bf16_to_f32(bits); }
uint16_t dgpp_f32_to_bf16(float v) { return f32_to_bf16(v); }
float dgpp_e4m3_to_f32(uint8_t code) { return e4m3_to_f32(code); }
uint8_t dgpp_f32_to_e4m3(float v) { return f32_to_e4m3(v); }
float dgpp_e2m1_to_f32(uint8_t code) { return e2m1_to_f32(code); }
uint8_t dgpp_f32_to_e2m1(float v) { return f32_to_e2m1(v); }
float dgpp_e8m0_to_f32(uint8_t code) { return e8m0_to_f32(code); }
uint8_t dgpp_e8m0_ceil_log2(float v) { return e8m0_ceil_log2(v); }

void dgpp_encode_fp8_blocks(const uint16_t* src_bf16, int64_t rows, int64_t cols, int block_rows, int block_cols,
                            uint8_t* payload, float* scales, int threads) {
  if (rows <= 0 || cols <= 0) return;
  const int64_t sr = (rows + block_rows - 1) / block_rows, sc = (cols + block_cols - 1) / block_cols;
  parallel_for(sr, threads, [&](int64_t b0, int64_t b1) {
    for (int64_t br = b0; br < b1; ++br)
      for (int64_t bc = 0; bc < sc; ++bc) {
        const int64_t r0 = br * block_rows, r1 = std::min(rows, r0 + block_rows);
        const int64_t c0 = bc * block_cols, c1 = std::min(cols, c0 + block_cols);
        float amax = 0.f;
        for (int64_t r = r0; r < r1; ++r)
          for (int64_t c = c0; c < c1; ++c) amax = std::max(amax, std::fabs(bf16_to_f32(src_bf16[r * cols + c])));
        const float s = amax > 0.f ? amax / 448.0f : 1.0f;
        scales[br * sc + bc] = s;
        for (int64_t r = r0; r < r1; ++r)
          for (int64_t c = c0; c < c1; ++c) payload[r * cols + c] = f32_to_e4m3(bf16_to_f32(src_bf16[r * cols + c]) / s);
      }
  });
}

float dgpp_encode_nvfp4(const float* src, int64_t rows, int64_t cols, uint8_t* payload, uint8_t* scales, int threads) {
  float amax = 0.f;
  for (int64_t i = 0; i < rows * cols; ++i) amax = std::max(amax, std::fabs(src[i]));
  const float ws2 = (amax > 0.f && std::isfinite(amax)) ? amax / (6.0f * 448.0f) : 1.0f;
  const int64_t groups = cols / 16;
  parallel_for(rows, threads, [&](int64_t r0, int64_t r1) {
    for (int64_t r = r0; r < r1; ++r)
      for (int64_t g = 0; g < groups; ++g) {
        const float* v = src + r * cols + g * 16;
        float bmax = 0.f;
        for (int j = 0; j < 16; ++j) bmax = std::max(bmax, std::fabs(v[j]));
        const uint8_t code = f32_to_e4m3(bmax / 6.0f / ws2);
        scales[r * groups + g] = code;
        const float S = e4m3_to_f32(code) * ws2;
        const float inv = S > 0.f ? 1.0f / S : 0.f;
        uint8_t* out = payload + (r * cols + g * 16) / 2;
        for (int j = 0; j < 16; j += 2)
          out[j / 2] = static_cast<uint8_t>(f32_to_e2m1(v[j] * inv) | (f32_to_e2m1(v[j + 1] * inv) << 4));
      }
  });
  return ws2;
}

void dgpp_encode_mxfp4(const float* src, int64_t rows, int64_t cols, uint8_t* payload, uint8_t* scales, int threads) {
  encode_mx_rows(src, rows, cols, 6.0f, scales, threads, [&](int64_t r, int64_t b, const float* v, float inv) {
    uint8_t* out = payload + (r * cols + b * 32) / 2;
    for (int j = 0; j < 32; j += 2)
      out[j / 2] = static_cast<uint8_t>(f32_to_e2m1(v[j] * inv) | (f32_to_e2m1(v[j + 1] * inv) << 4));
  });
}

void dgpp_encode_mxfp8(const float* src, int64_t rows, int64_t cols, uint8_t* payload, uint8_t* scales, int threads) {
  encode_mx_rows(src, rows, cols, 448.0f, scales, threads, [&](int64_t r, int64_t b, const float* v, float inv) {
    uint8_t* out = payload + r * cols + b * 32;
    for (int j = 0; j < 32; ++j) out[j] = f32_to_e4m3(v[j] * inv);
  });
}

void dgpp_fill_normal_f32(uint64_t seed, float mean, float stddev, int64_t n, float* out, int threads) {
  fill_normal(seed, mean, stddev, n, threads, [out](int64_t i, float v) { out[i] = v; });
}

void dgpp_fill_normal_bf16(uint64_t seed, float mean, float stddev, int64_t n, uint16_t* out, int threads) {
  fill_normal(seed, mean, stddev, n, threads, [out](int64_t i, float v) { out[i] = f32_to_bf16(v); });
}

void dgpp_fill_zipf_routes(uint64_t seed, double s, int tokens, int top_k, int n_experts, int32_t* ids) {
  std::vector<double> w(n_experts);
  for (int e = 0; e < n_experts; ++e) w[e] = 1.0 / std::pow(static_cast<double>(e + 1), s);
  std::vector<double> live(n_experts);
  for (int t = 0; t < tokens; ++t) {
    XorShift64 rng(block_seed(seed, static_cast<uint64_t>(t)));
    for (int i = 0; i < 8; ++i) rng.next();
    live = w;
    double total = 0;
    for (double v : live) total += v;
    int32_t* row = ids + static_cast<size_t>(t) * top_k;
    for (int j = 0; j < top_k; ++j) {  // sampling without replacement
      double u = rng.unit_open() * total, acc = 0;
      int pick = -1;
      for (int e = 0; e < n_experts; ++e) {
        if (live[e] <= 0) continue;
        acc += live[e];
        pick = e;
        if (acc >= u) break;
      }
      row[j] = pick;
      total -= live[pick];
      live[pick] = 0;
    }
    std::sort(row, row + top_k);
  }
}

}  // extern "C"
