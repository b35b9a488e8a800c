// Host side of the loader C ABI (include/dgpp_amd_loader.h): a memory-mapped safetensors reader and the
// pointer views over quantized matrices. No GPU calls.
//
// The header is scanned by a small strict JSON reader written for this one document shape: an object of
// tensor descriptors ({"dtype": string, "shape": [ints], "data_offsets": [begin, end]}) plus an optional
// "__metadata__" member that is kept as raw text. Everything the reference's reader rejects is rejected
// here with a message that names the same cause (src/loaders/safetensors.hpp:198-252; its unit tests
// tests/unit/safetensors_test.cpp:140-175 list the cases).
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <filesystem>
#include <fstream>
#include <iterator>
#include <map>
#include <set>
#include <cstdint>
#include <cstring>
#include <limits>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

#include "../../include/dgpp_amd_loader.h"

namespace {

thread_local std::string g_error;

int fail(int code, const std::string& msg) {
  g_error = msg;
  return code;
}

struct Tensor {
  std::string name;
  DgppTensorInfo info;
};

// ---- the JSON scanner -----------------------------------------------------------------------------------
struct Number {
  bool integer = false;   // an integer literal that fits int64
  int64_t value = 0;
};

class Scanner {
 public:
  explicit Scanner(std::string_view text) : s_(text) {}

  void ws() {
    while (p_ < s_.size() && (s_[p_] == ' ' || s_[p_] == '\t' || s_[p_] == '\n' || s_[p_] == '\r')) ++p_;
  }
  bool at_end() {
    ws();
    return p_ >= s_.size();
  }
  char peek() {
    ws();
    if (p_ >= s_.size()) throw std::runtime_error("unexpected end of header JSON");
    return s_[p_];
  }
  void expect(char c) {
    if (peek() != c) throw std::runtime_error(std::string("header JSON: expected '") + c + "'");
    ++p_;
  }
  bool take(char c) {
    if (peek() != c) return false;
    ++p_;
    return true;
  }

  std::string string() {
    expect('"');
    std::string out;
    while (true) {
      if (p_ >= s_.size()) throw std::runtime_error("header JSON: unterminated string");
      const unsigned char c = static_cast<unsigned char>(s_[p_++]);
      if (c == '"') return out;
      if (c < 0x20) throw std::runtime_error("header JSON: control character in string");
      if (c != '\\') {
        out.push_back(static_cast<char>(c));
        continue;
      }
      if (p_ >= s_.size()) throw std::runtime_error("header JSON: unterminated escape");
      const char e = s_[p_++];
      switch (e) {
        case '"': out.push_back('"'); break;
        case '\\': out.push_back('\\'); break;
        case '/': out.push_back('/'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'n': out.push_back('\n'); break;
        case 'r': out.push_back('\r'); break;
        case 't': out.push_back('\t'); break;
        case 'u': {
          unsigned cp = hex4();
          if (cp >= 0xD800 && cp <= 0xDBFF && p_ + 1 < s_.size() && s_[p_] == '\\' && s_[p_ + 1] == 'u') {
            p_ += 2;
            const unsigned lo = hex4();
            if (lo >= 0xDC00 && lo <= 0xDFFF) cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          }
          utf8(cp, out);
          break;
        }
        default: throw std::runtime_error("header JSON: bad escape");
      }
    }
  }

  // -?(0|[1-9][0-9]*)(.[0-9]+)?([eE][+-]?[0-9]+)?  — a leading zero before another digit is malformed.
  Number number() {
    ws();
    const size_t start = p_;
    bool neg = false;
    if (p_ < s_.size() && s_[p_] == '-') {
      neg = true;
      ++p_;
    }
    if (p_ >= s_.size() || s_[p_] < '0' || s_[p_] > '9') throw std::runtime_error("header JSON: malformed number");
    if (s_[p_] == '0' && p_ + 1 < s_.size() && s_[p_ + 1] >= '0' && s_[p_ + 1] <= '9')
      throw std::runtime_error("header JSON: malformed number (leading zero)");
    bool fits = true;
    uint64_t mag = 0;
    while (p_ < s_.size() && s_[p_] >= '0' && s_[p_] <= '9') {
      const uint64_t d = static_cast<uint64_t>(s_[p_] - '0');
      if (mag > (std::numeric_limits<uint64_t>::max() - d) / 10) fits = false;
      else mag = mag * 10 + d;
      ++p_;
    }
    bool integral = true;
    if (p_ < s_.size() && s_[p_] == '.') {
      integral = false;
      ++p_;
      if (p_ >= s_.size() || s_[p_] < '0' || s_[p_] > '9') throw std::runtime_error("header JSON: malformed number");
      while (p_ < s_.size() && s_[p_] >= '0' && s_[p_] <= '9') ++p_;
    }
    if (p_ < s_.size() && (s_[p_] == 'e' || s_[p_] == 'E')) {
      integral = false;
      ++p_;
      if (p_ < s_.size() && (s_[p_] == '+' || s_[p_] == '-')) ++p_;
      if (p_ >= s_.size() || s_[p_] < '0' || s_[p_] > '9') throw std::runtime_error("header JSON: malformed number");
      while (p_ < s_.size() && s_[p_] >= '0' && s_[p_] <= '9') ++p_;
    }
    (void)start;
    Number n;
    const uint64_t limit = neg ? (1ull << 63) : static_cast<uint64_t>(std::numeric_limits<int64_t>::max());
    if (integral && fits && mag <= limit) {
      n.integer = true;
      n.value = neg ? static_cast<int64_t>(0 - mag) : static_cast<int64_t>(mag);
    }
    return n;
  }

  void literal(const char* word) {
    ws();
    const size_t n = std::strlen(word);
    if (s_.compare(p_, n, word) != 0) throw std::runtime_error("header JSON: bad literal");
    p_ += n;
  }

  // Skips any value; returns its raw text.
  std::string_view skip_value() {
    ws();
    const size_t start = p_;
    skip();
    return s_.substr(start, p_ - start);
  }

 private:
  void skip() {
    const char c = peek();
    if (c == '{') {
      ++p_;
      if (take('}')) return;
      do {
        string();
        expect(':');
        skip();
      } while (take(','));
      expect('}');
    } else if (c == '[') {
      ++p_;
      if (take(']')) return;
      do skip();
      while (take(','));
      expect(']');
    } else if (c == '"') {
      string();
    } else if (c == 't') {
      literal("true");
    } else if (c == 'f') {
      literal("false");
    } else if (c == 'n') {
      literal("null");
    } else {
      number();
    }
  }
  unsigned hex4() {
    if (p_ + 4 > s_.size()) throw std::runtime_error("header JSON: bad \\u escape");
    unsigned v = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = s_[p_++];
      v <<= 4;
      if (c >= '0' && c <= '9') v |= static_cast<unsigned>(c - '0');
      else if (c >= 'a' && c <= 'f') v |= static_cast<unsigned>(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') v |= static_cast<unsigned>(c - 'A' + 10);
      else throw std::runtime_error("header JSON: bad \\u escape");
    }
    return v;
  }
  static void utf8(unsigned cp, std::string& out) {
    if (cp < 0x80) {
      out.push_back(static_cast<char>(cp));
    } else if (cp < 0x800) {
      out.push_back(static_cast<char>(0xC0 | (cp >> 6)));
      out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
      out.push_back(static_cast<char>(0xE0 | (cp >> 12)));
      out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
      out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    } else {
      out.push_back(static_cast<char>(0xF0 | (cp >> 18)));
      out.push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3F)));
      out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
      out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    }
  }

  std::string_view s_;
  size_t p_ = 0;
};

int dtype_of(std::string_view s) {
  if (s == "F32") return DGPP_DT_F32;
  if (s == "F16") return DGPP_DT_F16;
  if (s == "BF16") return DGPP_DT_BF16;
  if (s == "F8_E4M3" || s == "F8" || s == "FP8") return DGPP_DT_F8_E4M3;
  if (s == "I64") return DGPP_DT_I64;
  if (s == "I32") return DGPP_DT_I32;
  if (s == "U8" || s == "BOOL") return DGPP_DT_U8;
  if (s == "I8") return DGPP_DT_I8;
  if (s == "F8_E8M0") return DGPP_DT_F8_E8M0;
  if (s == "U32") return DGPP_DT_U32;
  if (s == "I16") return DGPP_DT_I16;
  return -1;
}

}  // namespace

struct DgppSafetensors {
  std::string path;
  int fd = -1;
  uint8_t* map = nullptr;
  size_t map_len = 0;
  uint64_t header_fold = 0;
  std::string metadata;
  std::vector<Tensor> tensors;   // sorted by name

  ~DgppSafetensors() { unmap(false); }

  void unmap(bool drop_page_cache) {
    if (map != nullptr) {
      munmap(map, map_len ? map_len : 1);
      map = nullptr;
    }
    if (fd >= 0) {
      if (drop_page_cache) posix_fadvise(fd, 0, 0, POSIX_FADV_DONTNEED);   // only effective after the munmap
      ::close(fd);
      fd = -1;
    }
    tensors.clear();
  }

  // One tensor descriptor; `s` stands on its '{'.
  void descriptor(Scanner& s, const std::string& name, uint64_t data_start) {
    bool have_dtype = false, have_shape = false, have_offsets = false;
    Tensor t;
    t.name = name;
    std::memset(&t.info, 0, sizeof(t.info));
    uint64_t begin = 0, end = 0;
    uint64_t numel = 1;
    s.expect('{');
    if (!s.take('}')) {
      do {
        const std::string key = s.string();
        s.expect(':');
        if (key == "dtype") {
          if (s.peek() != '"') throw std::runtime_error(path + ": tensor " + name + " dtype is not a string");
          const std::string d = s.string();
          const int dt = dtype_of(d);
          if (dt < 0) throw std::runtime_error(path + ": unknown dtype " + d);
          t.info.dtype = dt;
          have_dtype = true;
        } else if (key == "shape") {
          if (s.peek() != '[') throw std::runtime_error(path + ": tensor " + name + " shape is not an array");
          s.expect('[');
          int rank = 0;
          numel = 1;
          if (!s.take(']')) {
            do {
              const char c = s.peek();
              if (c != '-' && (c < '0' || c > '9'))
                throw std::runtime_error(path + ": tensor " + name + " shape must contain nonnegative integers");
              const Number n = s.number();
              if (!n.integer || n.value < 0)
                throw std::runtime_error(path + ": tensor " + name + " shape must contain nonnegative integers");
              if (rank >= DGPP_MAX_TENSOR_RANK)
                throw std::runtime_error(path + ": tensor " + name + " shape has more dimensions than this reader takes");
              t.info.shape[rank++] = n.value;
              // the ordered checked product: a zero met before an overflowing factor keeps the tensor empty,
              // a later zero does not undo an overflow
              const uint64_t d = static_cast<uint64_t>(n.value);
              if (numel != 0 && d > std::numeric_limits<size_t>::max() / numel)
                throw std::runtime_error(path + ": tensor " + name + " shape element count overflows");
              numel *= d;
            } while (s.take(','));
            s.expect(']');
          }
          t.info.rank = rank;
          have_shape = true;
        } else if (key == "data_offsets") {
          const std::string bad = path + ": tensor " + name + " data_offsets must contain two nonnegative integers";
          if (s.peek() != '[') throw std::runtime_error(bad);
          s.expect('[');
          uint64_t v[2] = {0, 0};
          int count = 0;
          if (!s.take(']')) {
            do {
              const char c = s.peek();
              if (c != '-' && (c < '0' || c > '9')) throw std::runtime_error(bad);
              const Number n = s.number();
              if (!n.integer || n.value < 0 || count >= 2) throw std::runtime_error(bad);
              v[count++] = static_cast<uint64_t>(n.value);
            } while (s.take(','));
            s.expect(']');
          }
          if (count != 2) throw std::runtime_error(bad);
          begin = v[0];
          end = v[1];
          have_offsets = true;
        } else {
          s.skip_value();
        }
      } while (s.take(','));
      s.expect('}');
    }
    if (!have_dtype) throw std::runtime_error(path + ": tensor " + name + " has no dtype");
    if (!have_shape) throw std::runtime_error(path + ": tensor " + name + " has no shape");
    if (!have_offsets) throw std::runtime_error(path + ": tensor " + name + " has no data_offsets");
    if (begin > end || end > map_len - data_start)
      throw std::runtime_error(path + ": tensor " + name + " has invalid data_offsets");
    const uint64_t width = dgpp_dtype_size(t.info.dtype);
    if (numel > std::numeric_limits<size_t>::max() / width || numel * width != end - begin)
      throw std::runtime_error(path + ": tensor " + name + " shape/dtype byte count mismatch");
    t.info.numel = numel;
    t.info.nbytes = end - begin;
    t.info.file_offset = data_start + begin;
    t.info.data = map + t.info.file_offset;
    // a name given twice: the later descriptor stands
    auto it = std::find_if(tensors.begin(), tensors.end(), [&](const Tensor& o) { return o.name == name; });
    if (it != tensors.end()) *it = std::move(t);
    else tensors.push_back(std::move(t));
  }

  void parse() {
    if (map_len < 8) throw std::runtime_error(path + ": too small for safetensors");
    uint64_t hlen;
    std::memcpy(&hlen, map, 8);
    if (hlen > map_len - 8) throw std::runtime_error(path + ": header length overruns file");
    const std::string_view json(reinterpret_cast<const char*>(map + 8), static_cast<size_t>(hlen));
    header_fold = 1469598103934665603ull;
    for (const char c : json) header_fold = (header_fold ^ static_cast<uint8_t>(c)) * 1099511628211ull;
    const uint64_t data_start = 8 + hlen;
    Scanner s(json);
    if (s.at_end() || s.peek() != '{') throw std::runtime_error(path + ": safetensors header not an object");
    s.expect('{');
    if (!s.take('}')) {
      do {
        const std::string key = s.string();
        s.expect(':');
        if (key == "__metadata__") {
          metadata = std::string(s.skip_value());
          continue;
        }
        if (s.peek() != '{') throw std::runtime_error(path + ": tensor " + key + " descriptor is not an object");
        descriptor(s, key, data_start);
      } while (s.take(','));
      s.expect('}');
    }
    if (!s.at_end()) throw std::runtime_error(path + ": trailing characters after the header object");
    std::sort(tensors.begin(), tensors.end(), [](const Tensor& a, const Tensor& b) { return a.name < b.name; });
  }

  void page_span(const DgppTensorInfo& t, size_t& begin, size_t& len) const {
    static const size_t page = static_cast<size_t>(sysconf(_SC_PAGESIZE));
    begin = static_cast<size_t>(t.file_offset / page) * page;
    size_t end = static_cast<size_t>((t.file_offset + t.nbytes + page - 1) / page) * page;
    if (end > map_len) end = map_len;
    len = end > begin ? end - begin : 0;
  }
};

extern "C" {

const char* dgpp_loader_last_error(void) { return g_error.c_str(); }

size_t dgpp_dtype_size(int dtype) {
  switch (dtype) {
    case DGPP_DT_F32: case DGPP_DT_I32: case DGPP_DT_U32: return 4;
    case DGPP_DT_F16: case DGPP_DT_BF16: case DGPP_DT_I16: return 2;
    case DGPP_DT_I64: return 8;
    case DGPP_DT_F8_E4M3: case DGPP_DT_U8: case DGPP_DT_I8: case DGPP_DT_F8_E8M0: return 1;
    default: return 0;
  }
}

int dgpp_safetensors_open(const char* path, DgppSafetensors** out) {
  if (!path || !out) return fail(DGPP_INVALID_ARGUMENT, "safetensors_open: null argument");
  *out = nullptr;
  DgppSafetensors* f = nullptr;
  try {
    f = new DgppSafetensors();
    f->path = path;
    f->fd = ::open(path, O_RDONLY | O_CLOEXEC);
    if (f->fd < 0) throw std::runtime_error(std::string("cannot open ") + path + ": " + std::strerror(errno));
    struct stat st {};
    if (fstat(f->fd, &st) != 0) throw std::runtime_error(std::string("fstat failed for ") + path);
    f->map_len = static_cast<size_t>(st.st_size);
    void* m = mmap(nullptr, f->map_len ? f->map_len : 1, PROT_READ, MAP_PRIVATE, f->fd, 0);
    if (m == MAP_FAILED) throw std::runtime_error(std::string("mmap failed for ") + path);
    f->map = static_cast<uint8_t*>(m);
    f->parse();
  } catch (const std::exception& e) {
    g_error = e.what();
    delete f;
    return DGPP_RUNTIME_ERROR;
  }
  *out = f;
  return DGPP_OK;
}

void dgpp_safetensors_close(DgppSafetensors* f, int drop_page_cache) {
  if (!f) return;
  f->unmap(drop_page_cache != 0);
  delete f;
}

int dgpp_safetensors_count(const DgppSafetensors* f) { return f ? static_cast<int>(f->tensors.size()) : 0; }

const char* dgpp_safetensors_name(const DgppSafetensors* f, int index) {
  if (!f || index < 0 || index >= static_cast<int>(f->tensors.size())) return nullptr;
  return f->tensors[static_cast<size_t>(index)].name.c_str();
}

int dgpp_safetensors_find(const DgppSafetensors* f, const char* name, DgppTensorInfo* out) {
  if (!f || !name || !out) return fail(DGPP_INVALID_ARGUMENT, "safetensors_find: null argument");
  const std::string_view key(name);
  auto it = std::lower_bound(f->tensors.begin(), f->tensors.end(), key,
                             [](const Tensor& t, std::string_view k) { return std::string_view(t.name) < k; });
  if (it == f->tensors.end() || it->name != key)
    return fail(DGPP_INVALID_ARGUMENT, "tensor not found: " + std::string(name) + " in " + f->path);
  *out = it->info;
  return DGPP_OK;
}

uint64_t dgpp_safetensors_header_fold(const DgppSafetensors* f) { return f ? f->header_fold : 0; }

const char* dgpp_safetensors_metadata_json(const DgppSafetensors* f) { return f ? f->metadata.c_str() : ""; }

void dgpp_safetensors_prefetch(const DgppSafetensors* f, const DgppTensorInfo* t) {
  if (!f || !t || f->map == nullptr || t->nbytes == 0) return;
  size_t begin, len;
  f->page_span(*t, begin, len);
  if (len) madvise(f->map + begin, len, MADV_WILLNEED);
}

void dgpp_safetensors_discard(const DgppSafetensors* f, const DgppTensorInfo* t) {
  if (!f || !t || f->map == nullptr || t->nbytes == 0) return;
  size_t begin, len;
  f->page_span(*t, begin, len);
  if (!len) return;
  madvise(f->map + begin, len, MADV_DONTNEED);
  posix_fadvise(f->fd, static_cast<off_t>(begin), static_cast<off_t>(len), POSIX_FADV_DONTNEED);
}

// ---- matrix views -----------------------------------------------------------------------------------------
int dgpp_quant_scale_shifts(const DgppQuantMatrix* m, int* rs, int* cs) {
  if (!m || !rs || !cs) return 0;
  auto log2_exact = [](int64_t v) {
    if (v <= 0 || (v & (v - 1)) != 0) return -1;
    int s = 0;
    while ((1LL << s) < v) ++s;
    return s;
  };
  *rs = log2_exact(m->scale_block_rows);
  *cs = log2_exact(m->scale_block_cols);
  return *rs >= 0 && *cs >= 4;
}

int dgpp_quant_rows_view(const DgppQuantMatrix* m, int64_t row_start, int64_t rows, DgppQuantMatrix* out) {
  if (!m || !out) return fail(DGPP_INVALID_ARGUMENT, "quant_rows_view: null argument");
  if (m->scale_block_rows <= 0 || m->scale_block_cols <= 0)
    return fail(DGPP_INVALID_ARGUMENT, "quant_rows_view: the scale block sizes must be positive");
  if (row_start < 0 || rows < 0 || rows > m->rows || row_start > m->rows - rows)
    return fail(DGPP_INVALID_ARGUMENT, "quant_rows_view: range out of bounds");
  if (row_start % m->scale_block_rows != 0)
    return fail(DGPP_INVALID_ARGUMENT,
                "quant_rows_view: row_start must be aligned to the scale block (a slice that starts inside a block "
                "cannot re-anchor the block scales)");
  const int64_t scale_cols = (m->cols + m->scale_block_cols - 1) / m->scale_block_cols;
  const int64_t first_block = row_start / m->scale_block_rows;
  DgppQuantMatrix v = *m;
  v.payload = m->payload + row_start * m->cols;
  v.scales = m->scales ? m->scales + first_block * scale_cols : nullptr;
  v.scales_e8m0 = m->scales_e8m0 ? m->scales_e8m0 + first_block * scale_cols : nullptr;
  v.rows = rows;
  *out = v;
  return DGPP_OK;
}

int dgpp_fp4_check_cols(int64_t cols, int scale_group) {
  if (scale_group != 16 && scale_group != 32) return fail(DGPP_INVALID_ARGUMENT, "fp4: the scale group must be 16 or 32");
  if (cols <= 0 || cols % scale_group != 0)
    return fail(DGPP_INVALID_ARGUMENT, "fp4: K must be a positive multiple of " + std::to_string(scale_group));
  return DGPP_OK;
}

int dgpp_fp4_rows_view(const DgppFp4Matrix* m, int64_t row_start, int64_t rows, DgppFp4Matrix* out) {
  if (!m || !out) return fail(DGPP_INVALID_ARGUMENT, "fp4_rows_view: null argument");
  const int rc = dgpp_fp4_check_cols(m->cols, m->scale_group);
  if (rc != DGPP_OK) return rc;
  if (row_start < 0 || rows < 0 || rows > m->rows || row_start > m->rows - rows)
    return fail(DGPP_INVALID_ARGUMENT, "fp4_rows_view: range out of bounds");
  DgppFp4Matrix v = *m;
  v.payload = m->payload + row_start * (m->cols / 2);
  v.scales = m->scales + row_start * (m->cols / m->scale_group);
  v.rows = rows;
  *out = v;
  return DGPP_OK;
}

namespace {
int64_t gcd64(int64_t a, int64_t b) {
  while (b != 0) {
    const int64_t t = a % b;
    a = b;
    b = t;
  }
  return a < 0 ? -a : a;
}
// The sliced axis' new block size, or 0 when the slice is not one this library takes.
int64_t slice_block(const DgppQuantMatrix* m, int axis, int64_t start, int64_t count) {
  if (!m || (axis != 0 && axis != 1) || m->scale_block_rows <= 0 || m->scale_block_cols <= 0) return 0;
  const int64_t extent = axis == 0 ? m->rows : m->cols;
  if (start < 0 || count <= 0 || count > extent || start > extent - count) return 0;
  const int64_t block = axis == 0 ? m->scale_block_rows : m->scale_block_cols;
  const int64_t g = gcd64(block, gcd64(start, count));
  if ((g & (g - 1)) != 0) return 0;
  if (g < 32 && g != block) return 0;   // the grid launchers take blocks of 32, 64 and 128 (or the parent's own)
  return g;
}
}  // namespace

int64_t dgpp_quant_slice_scale_count(const DgppQuantMatrix* m, int axis, int64_t start, int64_t count) {
  const int64_t g = slice_block(m, axis, start, count);
  if (g == 0) return -1;
  if (axis == 0) return ((count + g - 1) / g) * ((m->cols + m->scale_block_cols - 1) / m->scale_block_cols);
  return ((m->rows + m->scale_block_rows - 1) / m->scale_block_rows) * ((count + g - 1) / g);
}

int dgpp_quant_slice(const DgppQuantMatrix* m, int axis, int64_t start, int64_t count, uint8_t* payload_out,
                     float* scales_out, DgppQuantMatrix* out) {
  if (!m || !payload_out || !scales_out || !out) return fail(DGPP_INVALID_ARGUMENT, "quant_slice: null argument");
  if (!m->payload || !m->scales)
    return fail(DGPP_INVALID_ARGUMENT, "quant_slice: takes an E4M3 payload with an F32 scale grid (host addresses)");
  const int64_t g = slice_block(m, axis, start, count);
  if (g == 0)
    return fail(DGPP_INVALID_ARGUMENT,
                "quant_slice: the range must lie inside the matrix and re-block to a grid the launchers take "
                "(gcd(block, start, count) a power of two, at least 32 unless it is the parent's block)");
  const int64_t parent_cols = (m->cols + m->scale_block_cols - 1) / m->scale_block_cols;
  DgppQuantMatrix v = *m;
  v.payload = payload_out;
  v.scales = scales_out;
  v.scales_e8m0 = nullptr;
  if (axis == 0) {
    std::memcpy(payload_out, m->payload + start * m->cols, static_cast<size_t>(count * m->cols));
    const int64_t blocks = (count + g - 1) / g;
    for (int64_t i = 0; i < blocks; ++i) {
      const int64_t parent = (start + i * g) / m->scale_block_rows;
      std::memcpy(scales_out + i * parent_cols, m->scales + parent * parent_cols, static_cast<size_t>(parent_cols) * sizeof(float));
    }
    v.rows = count;
    v.scale_block_rows = static_cast<int32_t>(g);
  } else {
    for (int64_t r = 0; r < m->rows; ++r)
      std::memcpy(payload_out + r * count, m->payload + r * m->cols + start, static_cast<size_t>(count));
    const int64_t blocks = (count + g - 1) / g;
    const int64_t grid_rows = (m->rows + m->scale_block_rows - 1) / m->scale_block_rows;
    for (int64_t br = 0; br < grid_rows; ++br)
      for (int64_t j = 0; j < blocks; ++j)
        scales_out[br * blocks + j] = m->scales[br * parent_cols + (start + j * g) / m->scale_block_cols];
    v.cols = count;
    v.scale_block_cols = static_cast<int32_t>(g);
  }
  *out = v;
  return DGPP_OK;
}

int dgpp_fp4_cols_slice(const DgppFp4Matrix* m, int64_t col_start, int64_t cols, uint8_t* payload_out,
                        uint8_t* scales_out, DgppFp4Matrix* out) {
  if (!m || !payload_out || !scales_out || !out) return fail(DGPP_INVALID_ARGUMENT, "fp4_cols_slice: null argument");
  int rc = dgpp_fp4_check_cols(m->cols, m->scale_group);
  if (rc != DGPP_OK) return rc;
  rc = dgpp_fp4_check_cols(cols, m->scale_group);
  if (rc != DGPP_OK) return rc;
  if (!m->payload || !m->scales) return fail(DGPP_INVALID_ARGUMENT, "fp4_cols_slice: null payload or scales");
  if (col_start < 0 || col_start % m->scale_group != 0 || cols > m->cols || col_start > m->cols - cols)
    return fail(DGPP_INVALID_ARGUMENT, "fp4_cols_slice: the range must start on a scale-group boundary inside the matrix");
  const int64_t src_bytes = m->cols / 2, dst_bytes = cols / 2;
  const int64_t src_scales = m->cols / m->scale_group, dst_scales = cols / m->scale_group;
  for (int64_t r = 0; r < m->rows; ++r) {
    std::memcpy(payload_out + r * dst_bytes, m->payload + r * src_bytes + col_start / 2, static_cast<size_t>(dst_bytes));
    std::memcpy(scales_out + r * dst_scales, m->scales + r * src_scales + col_start / m->scale_group,
                static_cast<size_t>(dst_scales));
  }
  DgppFp4Matrix v = *m;
  v.payload = payload_out;
  v.scales = scales_out;
  v.cols = cols;
  *out = v;
  return DGPP_OK;
}

int dgpp_expert_view_from_quant(const DgppQuantMatrix* m, DgppMoeExpertView* out) {
  if (!m || !out) return fail(DGPP_INVALID_ARGUMENT, "expert_view_from_quant: null argument");
  int rs = 0, cs = 0;
  if (!m->payload || !m->scales)
    return fail(DGPP_INVALID_ARGUMENT, "expert_view_from_quant: the table takes E4M3 payloads with an F32 scale grid");
  if (!dgpp_quant_scale_shifts(m, &rs, &cs))
    return fail(DGPP_INVALID_ARGUMENT, "expert_view_from_quant: the scale blocks must be powers of two, columns >= 16");
  std::memset(out, 0, sizeof(*out));
  out->payload = m->payload;
  out->scales = m->scales;
  out->scale_shift_rows = rs;
  out->scale_shift_cols = cs;
  out->fp4_group = 16;
  return DGPP_OK;
}

int dgpp_expert_view_from_fp4(const DgppFp4Matrix* m, DgppMoeExpertView* out) {
  if (!m || !out) return fail(DGPP_INVALID_ARGUMENT, "expert_view_from_fp4: null argument");
  const int rc = dgpp_fp4_check_cols(m->cols, m->scale_group);
  if (rc != DGPP_OK) return rc;
  if (!m->payload || !m->scales) return fail(DGPP_INVALID_ARGUMENT, "expert_view_from_fp4: null payload or scales");
  if (m->scale_group == 16 && !m->global_scale)
    return fail(DGPP_INVALID_ARGUMENT, "expert_view_from_fp4: an NVFP4 matrix carries a device global scale");
  std::memset(out, 0, sizeof(*out));
  out->payload = m->payload;
  out->fp4_scales = m->scales;
  out->fp4_global = m->scale_group == 16 ? m->global_scale : nullptr;
  out->scale_shift_rows = 7;
  out->scale_shift_cols = 7;
  out->fp4_group = m->scale_group;
  return DGPP_OK;
}

}  // extern "C"

// ---- tensor names of a GLM-family MoE layer ------------------------------------------------------------------

namespace {

// The first of the shards that holds `name`, its description in `out`.
int find_in(const DgppSafetensors* const* files, int n_files, const std::string& name, DgppTensorInfo* out, int* file_index) {
  for (int i = 0; i < n_files; ++i) {
    if (!files[i]) continue;
    const std::string_view key(name);
    const auto& ts = files[i]->tensors;
    auto it = std::lower_bound(ts.begin(), ts.end(), key,
                               [](const Tensor& t, std::string_view k) { return std::string_view(t.name) < k; });
    if (it != ts.end() && it->name == key) {
      *out = it->info;
      if (file_index) *file_index = i;
      return DGPP_OK;
    }
  }
  return fail(DGPP_INVALID_ARGUMENT, "missing tensor '" + name + "'");
}

std::string shape_text(const DgppTensorInfo& t) {
  std::string s = "[";
  for (int i = 0; i < t.rank; ++i) s += (i ? ", " : "") + std::to_string(t.shape[i]);
  return s + "]";
}

int expect(const DgppTensorInfo& t, const std::string& name, int dtype, std::initializer_list<int64_t> shape) {
  bool ok = t.dtype == dtype && t.rank == static_cast<int>(shape.size());
  int i = 0;
  for (int64_t d : shape) ok = ok && t.shape[i++] == d;
  if (ok) return DGPP_OK;
  std::string want = "[";
  i = 0;
  for (int64_t d : shape) want += (i++ ? ", " : "") + std::to_string(d);
  return fail(DGPP_INVALID_ARGUMENT, "tensor '" + name + "' is dtype " + std::to_string(t.dtype) + " " + shape_text(t) +
                                         ", expected dtype " + std::to_string(dtype) + " " + want + "]");
}

// One logical [rows, cols] matrix named `base` ("...proj.weight"): the FP8 pair or the NVFP4 triple.
int bind_matrix(const DgppSafetensors* const* files, int n_files, const std::string& base, int64_t rows, int64_t cols, int format,
                DgppMoeMatrixTensors* out) {
  std::memset(out, 0, sizeof(*out));
  out->format = format;
  int rc;
  if (format == DGPP_BIND_NVFP4) {
    if (cols % 16 != 0) return fail(DGPP_INVALID_ARGUMENT, "NVFP4 needs K % 16 == 0: '" + base + "'");
    if ((rc = find_in(files, n_files, base + "_packed", &out->payload, &out->file_index)) != DGPP_OK) return rc;
    if ((rc = expect(out->payload, base + "_packed", DGPP_DT_U8, {rows, cols / 2})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, base + "_scale", &out->scales, nullptr)) != DGPP_OK) return rc;
    if ((rc = expect(out->scales, base + "_scale", DGPP_DT_F8_E4M3, {rows, cols / 16})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, base + "_global_scale", &out->global, nullptr)) != DGPP_OK) return rc;
    return expect(out->global, base + "_global_scale", DGPP_DT_F32, {1});
  }
  const std::string stem = base.size() > 7 && base.compare(base.size() - 7, 7, ".weight") == 0 ? base.substr(0, base.size() - 7) : base;
  if (format == DGPP_BIND_NVFP4_MODELOPT) {
    if (cols % 16 != 0) return fail(DGPP_INVALID_ARGUMENT, "NVFP4 needs K % 16 == 0: '" + base + "'");
    if ((rc = find_in(files, n_files, base, &out->payload, &out->file_index)) != DGPP_OK) return rc;
    if ((rc = expect(out->payload, base, DGPP_DT_U8, {rows, cols / 2})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_scale", &out->scales, nullptr)) != DGPP_OK) return rc;
    if ((rc = expect(out->scales, stem + ".weight_scale", DGPP_DT_F8_E4M3, {rows, cols / 16})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_scale_2", &out->global, nullptr)) != DGPP_OK) return rc;
    return expect(out->global, stem + ".weight_scale_2", DGPP_DT_F32, {});
  }
  if (format == DGPP_BIND_NVFP4_COMPRESSED) {
    if (cols % 16 != 0) return fail(DGPP_INVALID_ARGUMENT, "NVFP4 needs K % 16 == 0: '" + base + "'");
    if ((rc = find_in(files, n_files, stem + ".weight_packed", &out->payload, &out->file_index)) != DGPP_OK) return rc;
    if ((rc = expect(out->payload, stem + ".weight_packed", DGPP_DT_U8, {rows, cols / 2})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_scale", &out->scales, nullptr)) != DGPP_OK) return rc;
    if ((rc = expect(out->scales, stem + ".weight_scale", DGPP_DT_F8_E4M3, {rows, cols / 16})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_global_scale", &out->global, nullptr)) != DGPP_OK) return rc;
    return expect(out->global, stem + ".weight_global_scale", DGPP_DT_F32, {});
  }
  if (format == DGPP_BIND_MXFP4) {
    if (cols % 32 != 0) return fail(DGPP_INVALID_ARGUMENT, "MXFP4 needs K % 32 == 0: '" + base + "'");
    if ((rc = find_in(files, n_files, base, &out->payload, &out->file_index)) != DGPP_OK) return rc;
    if ((rc = expect(out->payload, base, DGPP_DT_U8, {rows, cols / 2})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_scale", &out->scales, nullptr)) != DGPP_OK) return rc;
    return expect(out->scales, stem + ".weight_scale", DGPP_DT_U8, {rows, cols / 32});
  }
  if (format == DGPP_BIND_MXFP8_SCALE_INV) {
    if (cols % 32 != 0) return fail(DGPP_INVALID_ARGUMENT, "MXFP8 needs K % 32 == 0: '" + base + "'");
    if ((rc = find_in(files, n_files, base, &out->payload, &out->file_index)) != DGPP_OK) return rc;
    if ((rc = expect(out->payload, base, DGPP_DT_F8_E4M3, {rows, cols})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_scale_inv", &out->scales, nullptr)) != DGPP_OK) return rc;
    return expect(out->scales, stem + ".weight_scale_inv", DGPP_DT_U8, {rows, cols / 32});
  }
  if (format == DGPP_BIND_MXFP8) {
    if (cols % 32 != 0) return fail(DGPP_INVALID_ARGUMENT, "MXFP8 needs K % 32 == 0: '" + base + "'");
    if ((rc = find_in(files, n_files, base, &out->payload, &out->file_index)) != DGPP_OK) return rc;
    if ((rc = expect(out->payload, base, DGPP_DT_F8_E4M3, {rows, cols})) != DGPP_OK) return rc;
    if ((rc = find_in(files, n_files, stem + ".weight_scale", &out->scales, nullptr)) != DGPP_OK) return rc;
    return expect(out->scales, stem + ".weight_scale", DGPP_DT_U8, {rows, cols / 32});
  }
  if (format != DGPP_BIND_FP8 && format != DGPP_BIND_FP8_BF16_SCALES)
    return fail(DGPP_INVALID_ARGUMENT, "unknown expert format " + std::to_string(format));
  if ((rc = find_in(files, n_files, base, &out->payload, &out->file_index)) != DGPP_OK) return rc;
  if ((rc = expect(out->payload, base, DGPP_DT_F8_E4M3, {rows, cols})) != DGPP_OK) return rc;
  if ((rc = find_in(files, n_files, base + "_scale_inv", &out->scales, nullptr)) != DGPP_OK) return rc;
  return expect(out->scales, base + "_scale_inv", format == DGPP_BIND_FP8 ? DGPP_DT_F32 : DGPP_DT_BF16,
                {(rows + 127) / 128, (cols + 127) / 128});
}

}  // namespace

extern "C" int dgpp_glm_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* layer_prefix, int n_experts,
                                       int64_t hidden, int64_t inter, int routed_format, int64_t shared_inter, int with_bias,
                                       DgppTensorInfo* router_weight, DgppTensorInfo* router_bias, DgppMoeMatrixTensors* shared,
                                       DgppMoeMatrixTensors* routed) {
  if (!files || n_files <= 0 || !layer_prefix || !router_weight || !routed || (shared_inter > 0 && !shared) || (with_bias && !router_bias))
    return fail(DGPP_INVALID_ARGUMENT, "glm_moe_bind_layer: null argument");
  if (n_experts <= 0 || hidden <= 0 || inter <= 0 || shared_inter < 0) return fail(DGPP_INVALID_ARGUMENT, "glm_moe_bind_layer: geometry must be positive");
  const std::string p(layer_prefix);
  static const char* const kProj[3] = {"gate_proj.weight", "up_proj.weight", "down_proj.weight"};
  int rc;
  if ((rc = find_in(files, n_files, p + "mlp.gate.weight", router_weight, nullptr)) != DGPP_OK) return rc;
  if ((rc = expect(*router_weight, p + "mlp.gate.weight", DGPP_DT_BF16, {n_experts, hidden})) != DGPP_OK) return rc;
  if (with_bias) {
    const std::string name = p + "mlp.gate.e_score_correction_bias";
    if ((rc = find_in(files, n_files, name, router_bias, nullptr)) != DGPP_OK) return rc;
    if ((rc = expect(*router_bias, name, DGPP_DT_F32, {n_experts})) != DGPP_OK) return rc;
  }
  if (shared_inter > 0) {
    // One shared expert under the un-indexed name, always block FP8.
    for (int m = 0; m < 3; ++m) {
      const int64_t rows = m == 2 ? hidden : shared_inter, cols = m == 2 ? shared_inter : hidden;
      if ((rc = bind_matrix(files, n_files, p + "mlp.shared_experts." + kProj[m], rows, cols, DGPP_BIND_FP8, shared + m)) != DGPP_OK)
        return rc;
    }
  }
  for (int e = 0; e < n_experts; ++e) {
    const std::string ep = p + "mlp.experts." + std::to_string(e) + ".";
    for (int m = 0; m < 3; ++m) {
      const int64_t rows = m == 2 ? hidden : inter, cols = m == 2 ? inter : hidden;
      if ((rc = bind_matrix(files, n_files, ep + kProj[m], rows, cols, routed_format, routed + static_cast<size_t>(e) * 3 + m)) !=
          DGPP_OK)
        return rc;
    }
  }
  return DGPP_OK;
}

extern "C" int dgpp_qwen_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* mlp_prefix, int n_experts,
                                        int64_t hidden, int64_t inter, int routed_format, int64_t shared_inter, int shared_format,
                                        DgppTensorInfo* router_weight, DgppTensorInfo* shared_gate, DgppMoeMatrixTensors* shared,
                                        DgppMoeMatrixTensors* routed) {
  if (!files || n_files <= 0 || !mlp_prefix || !router_weight || !routed || (shared_inter > 0 && (!shared || !shared_gate)))
    return fail(DGPP_INVALID_ARGUMENT, "qwen_moe_bind_layer: null argument");
  if (n_experts <= 0 || hidden <= 0 || inter <= 0 || shared_inter < 0)
    return fail(DGPP_INVALID_ARGUMENT, "qwen_moe_bind_layer: geometry must be positive");
  const std::string p(mlp_prefix);
  static const char* const kProj[3] = {"gate_proj.weight", "up_proj.weight", "down_proj.weight"};
  int rc;
  if ((rc = find_in(files, n_files, p + "gate.weight", router_weight, nullptr)) != DGPP_OK) return rc;
  if ((rc = expect(*router_weight, p + "gate.weight", DGPP_DT_BF16, {n_experts, hidden})) != DGPP_OK) return rc;
  if (shared_inter > 0) {
    if ((rc = find_in(files, n_files, p + "shared_expert_gate.weight", shared_gate, nullptr)) != DGPP_OK) return rc;
    if ((rc = expect(*shared_gate, p + "shared_expert_gate.weight", DGPP_DT_BF16, {1, hidden})) != DGPP_OK) return rc;
    for (int m = 0; m < 3; ++m) {
      const int64_t rows = m == 2 ? hidden : shared_inter, cols = m == 2 ? shared_inter : hidden;
      if ((rc = bind_matrix(files, n_files, p + "shared_expert." + kProj[m], rows, cols, shared_format, shared + m)) != DGPP_OK)
        return rc;
    }
  }
  for (int e = 0; e < n_experts; ++e) {
    const std::string ep = p + "experts." + std::to_string(e) + ".";
    for (int m = 0; m < 3; ++m) {
      const int64_t rows = m == 2 ? hidden : inter, cols = m == 2 ? inter : hidden;
      if ((rc = bind_matrix(files, n_files, ep + kProj[m], rows, cols, routed_format, routed + static_cast<size_t>(e) * 3 + m)) !=
          DGPP_OK)
        return rc;
    }
  }
  return DGPP_OK;
}

// src/models/mimo/binding.cpp:58-71: router BF16 + F32 bias, routed experts MXFP4, no shared expert.
extern "C" int dgpp_mimo_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* mlp_prefix, int n_experts,
                                        int64_t hidden, int64_t inter, DgppTensorInfo* router_weight, DgppTensorInfo* router_bias,
                                        DgppMoeMatrixTensors* routed) {
  if (!files || n_files <= 0 || !mlp_prefix || !router_weight || !router_bias || !routed)
    return fail(DGPP_INVALID_ARGUMENT, "mimo_moe_bind_layer: null argument");
  if (n_experts <= 0 || hidden <= 0 || inter <= 0) return fail(DGPP_INVALID_ARGUMENT, "mimo_moe_bind_layer: geometry must be positive");
  const std::string p(mlp_prefix);
  static const char* const kProj[3] = {"gate_proj.weight", "up_proj.weight", "down_proj.weight"};
  int rc;
  if ((rc = find_in(files, n_files, p + "gate.weight", router_weight, nullptr)) != DGPP_OK) return rc;
  if ((rc = expect(*router_weight, p + "gate.weight", DGPP_DT_BF16, {n_experts, hidden})) != DGPP_OK) return rc;
  if ((rc = find_in(files, n_files, p + "gate.e_score_correction_bias", router_bias, nullptr)) != DGPP_OK) return rc;
  if ((rc = expect(*router_bias, p + "gate.e_score_correction_bias", DGPP_DT_F32, {n_experts})) != DGPP_OK) return rc;
  for (int e = 0; e < n_experts; ++e) {
    const std::string ep = p + "experts." + std::to_string(e) + ".";
    for (int m = 0; m < 3; ++m) {
      const int64_t rows = m == 2 ? hidden : inter, cols = m == 2 ? inter : hidden;
      if ((rc = bind_matrix(files, n_files, ep + kProj[m], rows, cols, DGPP_BIND_MXFP4, routed + static_cast<size_t>(e) * 3 + m)) !=
          DGPP_OK)
        return rc;
    }
  }
  return DGPP_OK;
}

// src/models/minimax/binding.cpp:15-35, :60-71: F32 router and bias, the shared expert MXFP8 (`weight_scale_inv` bytes),
// routed experts NVFP4 under w1 (gate), w3 (up), w2 (down).
extern "C" int dgpp_minimax_moe_bind_layer(const DgppSafetensors* const* files, int n_files, const char* moe_prefix, int n_experts,
                                           int64_t hidden, int64_t inter, int64_t shared_inter, DgppTensorInfo* router_weight,
                                           DgppTensorInfo* router_bias, DgppMoeMatrixTensors* shared, DgppMoeMatrixTensors* routed) {
  if (!files || n_files <= 0 || !moe_prefix || !router_weight || !router_bias || !routed || (shared_inter > 0 && !shared))
    return fail(DGPP_INVALID_ARGUMENT, "minimax_moe_bind_layer: null argument");
  if (n_experts <= 0 || hidden <= 0 || inter <= 0 || shared_inter < 0)
    return fail(DGPP_INVALID_ARGUMENT, "minimax_moe_bind_layer: geometry must be positive");
  const std::string p(moe_prefix);
  static const char* const kProj[3] = {"gate_proj.weight", "up_proj.weight", "down_proj.weight"};
  static const char* const kW[3] = {"w1.weight", "w3.weight", "w2.weight"};
  int rc;
  if ((rc = find_in(files, n_files, p + "gate.weight", router_weight, nullptr)) != DGPP_OK) return rc;
  if ((rc = expect(*router_weight, p + "gate.weight", DGPP_DT_F32, {n_experts, hidden})) != DGPP_OK) return rc;
  if ((rc = find_in(files, n_files, p + "e_score_correction_bias", router_bias, nullptr)) != DGPP_OK) return rc;
  if ((rc = expect(*router_bias, p + "e_score_correction_bias", DGPP_DT_F32, {n_experts})) != DGPP_OK) return rc;
  for (int m = 0; m < 3 && shared_inter > 0; ++m) {
    const int64_t rows = m == 2 ? hidden : shared_inter, cols = m == 2 ? shared_inter : hidden;
    if ((rc = bind_matrix(files, n_files, p + "shared_experts." + kProj[m], rows, cols, DGPP_BIND_MXFP8_SCALE_INV, shared + m)) != DGPP_OK)
      return rc;
  }
  for (int e = 0; e < n_experts; ++e) {
    const std::string ep = p + "experts." + std::to_string(e) + ".";
    for (int m = 0; m < 3; ++m) {
      const int64_t rows = m == 2 ? hidden : inter, cols = m == 2 ? inter : hidden;
      if ((rc = bind_matrix(files, n_files, ep + kW[m], rows, cols, DGPP_BIND_NVFP4_COMPRESSED, routed + static_cast<size_t>(e) * 3 + m)) !=
          DGPP_OK)
        return rc;
    }
  }
  return DGPP_OK;
}

// ---- a checkpoint directory: the shard set and one name -> shard map ----------------------------------
struct DgppCheckpoint {
  std::vector<DgppSafetensors*> shards;            // in ascending path order
  std::map<std::string, int, std::less<>> where;   // tensor name -> index into shards
  ~DgppCheckpoint() {
    for (DgppSafetensors* f : shards) dgpp_safetensors_close(f, 0);
  }
};

int dgpp_checkpoint_open(const char* dir, DgppCheckpoint** out) {
  namespace fs = std::filesystem;
  if (!dir || !out) return fail(DGPP_INVALID_ARGUMENT, "checkpoint_open: null argument");
  *out = nullptr;
  DgppCheckpoint* ck = nullptr;
  try {
    const fs::path root(dir);
    if (!fs::is_directory(root)) throw std::runtime_error(std::string("checkpoint_open: not a directory: ") + dir);
    std::vector<fs::path> paths;
    const fs::path index_path = root / "model.safetensors.index.json";
    if (fs::exists(index_path)) {
      // The index's weight_map names the shard set, sub-directories included; a .safetensors file it does not
      // name is ignored (src/loaders/resident_stream.hpp:259-283).
      std::ifstream in(index_path, std::ios::binary);
      if (!in) throw std::runtime_error("checkpoint_open: cannot read shard index " + index_path.string());
      const std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
      std::set<std::string> named;
      bool have_map = false;
      Scanner s(text);
      s.expect('{');
      if (!s.take('}')) {
        do {
          const std::string key = s.string();
          s.expect(':');
          if (key != "weight_map") {
            s.skip_value();
            continue;
          }
          have_map = true;
          s.expect('{');
          if (!s.take('}')) {
            do {
              s.string();
              s.expect(':');
              if (s.peek() != '"') throw std::runtime_error("checkpoint_open: a weight_map entry is not a string");
              named.insert(s.string());
            } while (s.take(','));
            s.expect('}');
          }
        } while (s.take(','));
        s.expect('}');
      }
      if (!s.at_end()) throw std::runtime_error("checkpoint_open: trailing text after the shard index");
      if (!have_map) throw std::runtime_error("checkpoint_open: the shard index has no weight_map");
      for (const std::string& name : named) {
        const fs::path f = root / name;
        if (!fs::exists(f))
          throw std::runtime_error("checkpoint_open: shard '" + name + "' named by the index is missing from " + dir);
        paths.push_back(f);
      }
    } else {
      for (const auto& entry : fs::directory_iterator(root))
        if (entry.path().extension() == ".safetensors") paths.push_back(entry.path());
    }
    if (paths.empty()) throw std::runtime_error(std::string("checkpoint_open: no .safetensors shards in ") + dir);
    std::sort(paths.begin(), paths.end());
    ck = new DgppCheckpoint();
    for (const fs::path& f : paths) {
      DgppSafetensors* h = nullptr;
      if (dgpp_safetensors_open(f.string().c_str(), &h) != DGPP_OK) throw std::runtime_error(g_error);
      ck->shards.push_back(h);
      const int at = static_cast<int>(ck->shards.size()) - 1;
      for (const Tensor& t : h->tensors)
        if (!ck->where.emplace(t.name, at).second)
          throw std::runtime_error("checkpoint_open: duplicate tensor '" + t.name + "' in " + f.string());
    }
  } catch (const std::exception& e) {
    const std::string msg = e.what();   // the shards' closes below do not touch it, but keep it safe
    delete ck;
    g_error = msg;
    return DGPP_RUNTIME_ERROR;
  }
  *out = ck;
  return DGPP_OK;
}

void dgpp_checkpoint_close(DgppCheckpoint* ck) { delete ck; }

int dgpp_checkpoint_shard_count(const DgppCheckpoint* ck) { return ck ? static_cast<int>(ck->shards.size()) : 0; }

const DgppSafetensors* const* dgpp_checkpoint_shards(const DgppCheckpoint* ck) {
  return ck && !ck->shards.empty() ? ck->shards.data() : nullptr;
}

const char* dgpp_checkpoint_shard_path(const DgppCheckpoint* ck, int index) {
  if (!ck || index < 0 || index >= static_cast<int>(ck->shards.size())) return nullptr;
  return ck->shards[static_cast<size_t>(index)]->path.c_str();
}

uint64_t dgpp_checkpoint_tensor_count(const DgppCheckpoint* ck) { return ck ? ck->where.size() : 0; }

int dgpp_checkpoint_find(const DgppCheckpoint* ck, const char* name, DgppTensorInfo* out, int* shard_index) {
  if (!ck || !name || !out) return fail(DGPP_INVALID_ARGUMENT, "checkpoint_find: null argument");
  const auto it = ck->where.find(std::string_view(name));
  if (it == ck->where.end()) return fail(DGPP_INVALID_ARGUMENT, std::string("missing tensor '") + name + "'");
  if (shard_index) *shard_index = it->second;
  return dgpp_safetensors_find(ck->shards[static_cast<size_t>(it->second)], name, out);
}
