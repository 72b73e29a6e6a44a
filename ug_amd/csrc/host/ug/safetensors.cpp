#include "safetensors.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cmath>
#include <algorithm>
#include <cerrno>
#include <cstdlib>
#include <cstring>
#include <limits>

namespace ug {

namespace {

// ---- a JSON reader for the header: objects, arrays, strings, non-negative integers ----------------
struct Json {
  enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
  double num = 0;
  bool is_uint = false;
  uint64_t uint = 0;
  std::string str;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;
};

struct JsonParser {
  const char* p;
  const char* end;
  const std::string& path;
  [[noreturn]] void fail(const std::string& what) const { bail("invalid safetensors header in " + path + ": " + what); }
  void ws() {
    while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p;
  }
  char peek() {
    ws();
    if (p >= end) fail("unexpected end");
    return *p;
  }
  void expect(char c) {
    if (peek() != c) fail(std::string("expected '") + c + "'");
    ++p;
  }
  std::string string() {
    expect('"');
    std::string out;
    while (true) {
      if (p >= end) fail("unterminated string");
      char c = *p++;
      if (c == '"') break;
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (p >= end) fail("unterminated escape");
      char e = *p++;
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
          if (end - p < 4) fail("short \\u escape");
          unsigned cp = 0;
          for (int i = 0; i < 4; ++i) {
            char h = *p++;
            cp <<= 4;
            if (h >= '0' && h <= '9') cp |= (unsigned)(h - '0');
            else if (h >= 'a' && h <= 'f') cp |= (unsigned)(h - 'a' + 10);
            else if (h >= 'A' && h <= 'F') cp |= (unsigned)(h - 'A' + 10);
            else fail("bad \\u escape");
          }
          // UTF-8 encode the BMP code point (surrogate pairs are kept as two 3-byte sequences)
          if (cp < 0x80) out.push_back((char)cp);
          else if (cp < 0x800) {
            out.push_back((char)(0xC0 | (cp >> 6)));
            out.push_back((char)(0x80 | (cp & 0x3F)));
          } else {
            out.push_back((char)(0xE0 | (cp >> 12)));
            out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
            out.push_back((char)(0x80 | (cp & 0x3F)));
          }
          break;
        }
        default: fail("bad escape");
      }
    }
    return out;
  }
  Json value(int depth) {
    if (depth > 16) fail("nesting too deep");
    Json j;
    char c = peek();
    if (c == '{') {
      ++p;
      j.kind = Json::Obj;
      if (peek() == '}') {
        ++p;
        return j;
      }
      while (true) {
        std::string k = string();
        expect(':');
        j.obj.emplace_back(std::move(k), value(depth + 1));
        char d = peek();
        ++p;
        if (d == '}') break;
        if (d != ',') fail("expected ',' or '}'");
        ws();
      }
    } else if (c == '[') {
      ++p;
      j.kind = Json::Arr;
      if (peek() == ']') {
        ++p;
        return j;
      }
      while (true) {
        j.arr.push_back(value(depth + 1));
        char d = peek();
        ++p;
        if (d == ']') break;
        if (d != ',') fail("expected ',' or ']'");
      }
    } else if (c == '"') {
      j.kind = Json::Str;
      j.str = string();
    } else if (c == 't' && end - p >= 4 && !strncmp(p, "true", 4)) {
      p += 4;
      j.kind = Json::Bool;
      j.num = 1;
    } else if (c == 'f' && end - p >= 5 && !strncmp(p, "false", 5)) {
      p += 5;
      j.kind = Json::Bool;
    } else if (c == 'n' && end - p >= 4 && !strncmp(p, "null", 4)) {
      p += 4;
    } else if (c == '-' || (c >= '0' && c <= '9')) {
      const char* s = p;
      bool all_digits = true;
      uint64_t u = 0;
      bool overflow = false;
      while (p < end && (*p == '-' || *p == '+' || *p == '.' || *p == 'e' || *p == 'E' || (*p >= '0' && *p <= '9'))) {
        if (*p >= '0' && *p <= '9') {
          if (u > (std::numeric_limits<uint64_t>::max() - (uint64_t)(*p - '0')) / 10) overflow = true;
          u = u * 10 + (uint64_t)(*p - '0');
        } else {
          all_digits = false;
        }
        ++p;
      }
      j.kind = Json::Num;
      j.num = strtod(std::string(s, p).c_str(), nullptr);
      j.is_uint = all_digits && !overflow;
      j.uint = u;
    } else {
      fail(std::string("unexpected character '") + c + "'");
    }
    return j;
  }
};

size_t st_dtype_size(const std::string& d) {
  if (d == "BOOL" || d == "U8" || d == "I8" || d == "F8_E5M2" || d == "F8_E4M3") return 1;
  if (d == "I16" || d == "U16" || d == "F16" || d == "BF16") return 2;
  if (d == "I32" || d == "U32" || d == "F32") return 4;
  if (d == "I64" || d == "U64" || d == "F64") return 8;
  return 0;
}

// safetensors.rs:89-96
DType ug_dtype(const std::string& st_dtype, const std::string& name) {
  if (st_dtype == "BF16") return DType::BF16;
  if (st_dtype == "F16") return DType::F16;
  if (st_dtype == "F32") return DType::F32;
  if (st_dtype == "I32") return DType::I32;
  if (st_dtype == "I64") return DType::I64;
  bail("unsupported dtype for " + name + ": " + st_dtype);
}

}  // namespace

struct MmapedSafetensors::File {
  std::string path;
  void* map = nullptr;
  size_t len = 0;
  std::vector<std::pair<std::string, TensorView>> tensors;  // in header order
  std::map<std::string, size_t> index;
  ~File() {
    if (map) munmap(map, len);
  }
};

std::shared_ptr<MmapedSafetensors::File> MmapedSafetensors::open_file(const std::string& path) {
  auto f = std::make_shared<MmapedSafetensors::File>();
  f->path = path;
  int fd = ::open(path.c_str(), O_RDONLY);
  if (fd < 0) bail(std::string(strerror(errno)) + ", path: " + path);
  struct stat st;
  if (fstat(fd, &st) != 0) {
    int e = errno;
    close(fd);
    bail(std::string(strerror(e)) + ", path: " + path);
  }
  f->len = (size_t)st.st_size;
  if (f->len < 8) {
    close(fd);
    bail("safetensors header too small, path: " + path);
  }
  f->map = mmap(nullptr, f->len, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (f->map == MAP_FAILED) {
    f->map = nullptr;
    bail(std::string("mmap failed: ") + strerror(errno) + ", path: " + path);
  }
  const uint8_t* base = static_cast<const uint8_t*>(f->map);
  uint64_t n = 0;
  for (int i = 7; i >= 0; --i) n = (n << 8) | base[i];
  if (n > 100000000ull) bail("safetensors header too large, path: " + path);
  if (n + 8 > f->len) bail("invalid safetensors header length, path: " + path);
  const char* hs = reinterpret_cast<const char*>(base + 8);
  JsonParser jp{hs, hs + n, path};
  Json root = jp.value(0);
  jp.ws();
  if (jp.p != jp.end) jp.fail("trailing characters");
  if (root.kind != Json::Obj) jp.fail("the header is not an object");
  const uint8_t* data = base + 8 + n;
  const size_t data_len = f->len - 8 - (size_t)n;
  std::vector<std::pair<size_t, size_t>> spans;
  for (auto& kv : root.obj) {
    if (kv.first == "__metadata__") {
      if (kv.second.kind != Json::Obj) jp.fail("__metadata__ is not an object");
      for (auto& m : kv.second.obj)
        if (m.second.kind != Json::Str) jp.fail("__metadata__ values must be strings");
      continue;
    }
    const Json& t = kv.second;
    if (t.kind != Json::Obj) jp.fail("tensor entry " + kv.first + " is not an object");
    TensorView v;
    bool have_shape = false, have_off = false;
    size_t begin = 0, end = 0;
    for (auto& fld : t.obj) {
      if (fld.first == "dtype" && fld.second.kind == Json::Str) {
        v.dtype = fld.second.str;
      } else if (fld.first == "shape" && fld.second.kind == Json::Arr) {
        for (const Json& d : fld.second.arr) {
          if (d.kind != Json::Num || !d.is_uint) jp.fail("bad shape for " + kv.first);
          v.shape.push_back((size_t)d.uint);
        }
        have_shape = true;
      } else if (fld.first == "data_offsets" && fld.second.kind == Json::Arr && fld.second.arr.size() == 2 && fld.second.arr[0].is_uint &&
                 fld.second.arr[1].is_uint) {
        begin = (size_t)fld.second.arr[0].uint;
        end = (size_t)fld.second.arr[1].uint;
        have_off = true;
      }
    }
    const size_t esz = st_dtype_size(v.dtype);
    if (!esz || !have_shape || !have_off) jp.fail("incomplete entry for " + kv.first);
    if (begin > end || end > data_len) jp.fail("invalid offsets for " + kv.first);
    size_t n_el = 1;
    for (size_t d : v.shape) {
      if (d && n_el > std::numeric_limits<size_t>::max() / d) jp.fail("shape overflow for " + kv.first);
      n_el *= d;
    }
    if (n_el > std::numeric_limits<size_t>::max() / esz || n_el * esz != end - begin) jp.fail("tensor " + kv.first + ": shape and data_offsets disagree");
    v.data = data + begin;
    v.nbytes = end - begin;
    spans.push_back({begin, end});
    if (f->index.count(kv.first)) jp.fail("duplicate tensor " + kv.first);
    f->index[kv.first] = f->tensors.size();
    f->tensors.emplace_back(kv.first, std::move(v));
  }
  // the crate requires the tensors to tile the data section without holes or overlaps
  std::sort(spans.begin(), spans.end());
  size_t at = 0;
  for (auto& s : spans) {
    if (s.first != at) jp.fail("invalid offsets: tensors do not tile the data section");
    at = s.second;
  }
  if (at != data_len) jp.fail("data section is longer than the tensors it holds");
  return f;
}

MmapedSafetensors MmapedSafetensors::open(const std::string& path) {
  MmapedSafetensors s;
  s.files_.push_back(open_file(path));
  return s;
}

MmapedSafetensors MmapedSafetensors::multi(const std::vector<std::string>& paths) {
  MmapedSafetensors s;
  s.routed_ = true;
  for (size_t i = 0; i < paths.size(); ++i) {
    s.files_.push_back(open_file(paths[i]));
    for (auto& kv : s.files_.back()->tensors) s.routing_[kv.first] = i;
  }
  return s;
}

std::vector<std::pair<std::string, TensorView>> MmapedSafetensors::tensors() const {
  std::vector<std::pair<std::string, TensorView>> out;
  for (auto& f : files_)
    for (auto& kv : f->tensors) out.push_back(kv);
  return out;
}

TensorView MmapedSafetensors::get(const std::string& name) const {
  size_t idx = 0;
  if (routed_) {
    auto it = routing_.find(name);
    if (it == routing_.end()) bail("cannot find tensor " + name);
    idx = it->second;
  }
  if (idx >= files_.size()) bail("cannot find tensor " + name);
  const File& f = *files_[idx];
  auto it = f.index.find(name);
  if (it == f.index.end()) bail("cannot find tensor " + name + " in " + f.path);
  return f.tensors[it->second].second;
}

std::pair<Shape, std::unique_ptr<Slice>> MmapedSafetensors::load_slice(const std::string& name, const DevicePtr& dev) const {
  TensorView v = get(name);
  Shape shape(v.shape);
  DType dt = ug_dtype(v.dtype, name);
  std::unique_ptr<Slice> slice = dev->allocate_uninit(dt, shape.num_elements());
  // the upload takes any alignment (the reference copies into an aligned Vec first when needed, :297-318)
  if (shape.num_elements()) slice->copy_host_to_device(v.data, dt, shape.num_elements());
  return {shape, std::move(slice)};
}

std::pair<Shape, std::unique_ptr<Slice>> MmapedSafetensors::load_slice_with_cast(const std::string& name, DType dst_dtype, const DevicePtr& dev) const {
  TensorView v = get(name);
  Shape shape(v.shape);
  DType src_dtype = ug_dtype(v.dtype, name);
  if (src_dtype == dst_dtype) return load_slice(name, dev);
  const size_t n = shape.num_elements();
  // safetensors.rs:161-165, 187-191: these two arms build a Vec<i32> for an I64 slice, which the
  // upload then rejects.
  if (dst_dtype == DType::I64 && (src_dtype == DType::BF16 || src_dtype == DType::F16))
    bail(std::string("dtype mismatch in copy_host_to_device, dst I64, src I32 (loading ") + name + " with cast " + dtype_str(src_dtype) + " -> I64)");
  std::unique_ptr<Slice> dst = dev->allocate_uninit(dst_dtype, n);
  last_cast_on_device_ = false;
  if (n == 0) return {shape, std::move(dst)};
  // UG_SAFETENSORS_HOST_CAST=1 forces the reference's order (convert on the host, then upload).
  if (!getenv("UG_SAFETENSORS_HOST_CAST")) {
    std::unique_ptr<Slice> staged = dev->allocate_uninit(src_dtype, n);
    staged->copy_host_to_device(v.data, src_dtype, n);
    if (dev->convert(*dst, *staged)) {
      last_cast_on_device_ = true;
      return {shape, std::move(dst)};
    }
  }
  std::vector<uint8_t> host(n * size_in_bytes(dst_dtype));
  convert_on_host(v.data, src_dtype, host.data(), dst_dtype, n, name);
  dst->copy_host_to_device(host.data(), dst_dtype, n);
  return {shape, std::move(dst)};
}

LazyBuffer MmapedSafetensors::load(const std::string& name, const DevicePtr& dev) const {
  auto r = load_slice(name, dev);
  return LazyBuffer::from_slice(std::move(r.second), r.first, dev);
}

LazyBuffer MmapedSafetensors::load_with_cast(const std::string& name, DType dtype, const DevicePtr& dev) const {
  auto r = load_slice_with_cast(name, dtype, dev);
  return LazyBuffer::from_slice(std::move(r.second), r.first, dev);
}

// ---- host conversions (half 2.x semantics for the 16-bit floats, Rust `as` for the integers) ----------
namespace {

int32_t f32_as_i32(float f) {
  if (f != f) return 0;
  if (f >= 2147483648.f) return std::numeric_limits<int32_t>::max();
  if (f <= -2147483648.f) return std::numeric_limits<int32_t>::min();
  return (int32_t)f;
}
int64_t f32_as_i64(float f) {
  if (f != f) return 0;
  if (f >= 9223372036854775808.f) return std::numeric_limits<int64_t>::max();
  if (f <= -9223372036854775808.f) return std::numeric_limits<int64_t>::min();
  return (int64_t)f;
}

template <typename T>
T load_unaligned(const uint8_t* p, size_t i) {
  T v;
  memcpy(&v, p + i * sizeof(T), sizeof(T));
  return v;
}

float src_as_f32(const uint8_t* src, DType dt, size_t i) {
  switch (dt) {
    case DType::BF16: return bf16_bits_to_f32(load_unaligned<uint16_t>(src, i));
    case DType::F16: return f16_bits_to_f32(load_unaligned<uint16_t>(src, i));
    case DType::F32: return load_unaligned<float>(src, i);
    case DType::I32: return (float)load_unaligned<int32_t>(src, i);
    case DType::I64: return (float)load_unaligned<int64_t>(src, i);
  }
  return 0.f;
}

}  // namespace

void convert_on_host(const uint8_t* src, DType sd, void* dst, DType dd, size_t n, const std::string& name) {
  if (dd == DType::I64 && (sd == DType::BF16 || sd == DType::F16)) bail("dtype mismatch in copy_host_to_device, dst I64, src I32 (loading " + name + ")");
  for (size_t i = 0; i < n; ++i) {
    if (sd == dd) {
      memcpy(static_cast<uint8_t*>(dst) + i * size_in_bytes(dd), src + i * size_in_bytes(sd), size_in_bytes(dd));
      continue;
    }
    if (sd == DType::I32 && dd == DType::I64) {
      static_cast<int64_t*>(dst)[i] = (int64_t)load_unaligned<int32_t>(src, i);
      continue;
    }
    if (sd == DType::I64 && dd == DType::I32) {
      static_cast<int32_t*>(dst)[i] = (int32_t)(uint32_t)(uint64_t)load_unaligned<int64_t>(src, i);
      continue;
    }
    const float f = src_as_f32(src, sd, i);
    switch (dd) {
      case DType::BF16: static_cast<uint16_t*>(dst)[i] = f32_to_bf16_bits(f); break;
      case DType::F16: static_cast<uint16_t*>(dst)[i] = f32_to_f16_bits(f); break;
      case DType::F32: static_cast<float*>(dst)[i] = f; break;
      case DType::I32: static_cast<int32_t*>(dst)[i] = f32_as_i32(f); break;
      case DType::I64: static_cast<int64_t*>(dst)[i] = f32_as_i64(f); break;
    }
  }
}

}  // namespace ug
