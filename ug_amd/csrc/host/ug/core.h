// Data model shared by the host-side front-end: errors, dtypes, constants, shapes, layouts.
// Mirrors ug-core/src/{error,dtype,const,layout}.rs.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "ughip.h"

namespace ug {

// ug::Error (ug-core/src/error.rs:3-100): every failure on the path is a message.
struct Error : std::runtime_error {
  explicit Error(const std::string& m) : std::runtime_error(m) {}
};

[[noreturn]] inline void bail(const std::string& m) { throw Error(m); }

// ug::DType (dtype.rs:5-59); numeric values are the wire values of include/ughip.h.
enum class DType : int { BF16 = UGHIP_BF16, F16 = UGHIP_F16, F32 = UGHIP_F32, I32 = UGHIP_I32, I64 = UGHIP_I64 };

inline size_t size_in_bytes(DType d) {
  switch (d) {
    case DType::BF16:
    case DType::F16: return 2;
    case DType::F32:
    case DType::I32: return 4;
    case DType::I64: return 8;
  }
  return 0;
}

inline const char* dtype_str(DType d) {
  switch (d) {
    case DType::BF16: return "BF16";
    case DType::F16: return "F16";
    case DType::F32: return "F32";
    case DType::I32: return "I32";
    case DType::I64: return "I64";
  }
  return "?";
}

inline bool is_float(DType d) { return d == DType::BF16 || d == DType::F16 || d == DType::F32; }

// Round-to-nearest-even f32 -> bf16 bits and back (half::bf16::from_f32).
inline uint16_t f32_to_bf16_bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN stays NaN
  uint32_t round = 0x7fffu + ((u >> 16) & 1);
  return (uint16_t)((u + round) >> 16);
}
inline float bf16_bits_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// IEEE binary16 <-> f32 (half::f16::{to_f32, from_f32}: round to nearest even).
inline float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else {  // subnormal: normalise
      int e = -1;
      uint32_t m = man;
      do {
        ++e;
        m <<= 1;
      } while ((m & 0x400u) == 0);
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
inline uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t man = x & 0x007fffffu;
  const int32_t exp = (int32_t)((x >> 23) & 0xff);
  if (exp == 255) return (uint16_t)(sign | 0x7c00u | (man ? (0x0200u | (man >> 13)) : 0));
  const int32_t half_exp = exp - 127 + 15;
  if (half_exp >= 31) return (uint16_t)(sign | 0x7c00u);
  if (half_exp <= 0) {
    if (14 - half_exp > 24) return (uint16_t)sign;
    const uint32_t m = man | 0x00800000u;
    const int shift = 14 - half_exp;
    uint32_t half_man = m >> shift;
    const uint32_t round_bit = 1u << (shift - 1);
    if ((m & round_bit) != 0 && (m & (3 * round_bit - 1)) != 0) half_man += 1;
    return (uint16_t)(sign | half_man);
  }
  uint32_t out = sign | ((uint32_t)half_exp << 10) | (man >> 13);
  const uint32_t round_bit = 0x00001000u;
  if ((man & round_bit) != 0 && (man & (3 * round_bit - 1)) != 0) out += 1;  // may carry into the exponent: correct
  return (uint16_t)out;
}
// ug::Const (const.rs:83-174): a typed scalar; floats may not be NaN.
struct Const {
  DType dtype = DType::F32;
  int64_t i = 0;
  float f = 0.f;

  static Const f32(float v) {
    if (std::isnan(v)) bail("cannot use nan in const");
    Const c;
    c.dtype = DType::F32;
    c.f = v;
    return c;
  }
  static Const bf16(float v) {
    if (std::isnan(v)) bail("cannot use nan in const");
    Const c;
    c.dtype = DType::BF16;
    c.f = bf16_bits_to_f32(f32_to_bf16_bits(v));
    return c;
  }
  static Const i32(int32_t v) {
    Const c;
    c.dtype = DType::I32;
    c.i = v;
    return c;
  }
  static Const i64(int64_t v) {
    Const c;
    c.dtype = DType::I64;
    c.i = v;
    return c;
  }
  static Const zero(DType d) {
    Const c;
    c.dtype = d;
    return c;
  }
  // const.rs:155-173: floats use -inf / +inf.
  static Const min_value(DType d) {
    Const c;
    c.dtype = d;
    if (is_float(d)) c.f = -INFINITY;
    else c.i = d == DType::I32 ? INT32_MIN : INT64_MIN;
    return c;
  }
  static Const max_value(DType d) {
    Const c;
    c.dtype = d;
    if (is_float(d)) c.f = INFINITY;
    else c.i = d == DType::I32 ? INT32_MAX : INT64_MAX;
    return c;
  }
  bool operator==(const Const& o) const {
    return dtype == o.dtype && i == o.i && std::memcmp(&f, &o.f, 4) == 0;
  }
  std::string key() const {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    char buf[64];
    snprintf(buf, sizeof buf, "c%d:%lld:%08x", (int)dtype, (long long)i, u);
    return buf;
  }
};

// ug::Shape (layout.rs:5-85).
struct Shape {
  std::vector<size_t> dims_;
  Shape() = default;
  Shape(std::vector<size_t> d) : dims_(std::move(d)) {}
  Shape(std::initializer_list<size_t> d) : dims_(d) {}
  const std::vector<size_t>& dims() const { return dims_; }
  size_t rank() const { return dims_.size(); }
  size_t num_elements() const {
    size_t n = 1;
    for (size_t d : dims_) n *= d;
    return n;
  }
  size_t elem_count() const { return num_elements(); }
  std::vector<size_t> stride_contiguous() const {
    std::vector<size_t> s(dims_.size());
    size_t st = 1;
    for (size_t k = dims_.size(); k-- > 0;) {
      s[k] = st;
      st *= dims_[k];
    }
    return s;
  }
  bool operator==(const Shape& o) const { return dims_ == o.dims_; }
  bool operator!=(const Shape& o) const { return dims_ != o.dims_; }
  std::string str() const {
    std::string s = "[";
    for (size_t k = 0; k < dims_.size(); ++k) s += (k ? ", " : "") + std::to_string(dims_[k]);
    return s + "]";
  }
};

// Dim::to_index with D::Minus1 / D::Minus2 (layout.rs:226-307): negative values count from the end.
inline size_t dim_index(long dim, const Shape& shape, const char* op) {
  long r = (long)shape.rank();
  long d = dim < 0 ? r + dim : dim;
  if (d < 0 || d >= r) bail(std::string(op) + ": dim " + std::to_string(dim) + " out of range for shape " + shape.str());
  return (size_t)d;
}

// ug::Layout (layout.rs:577-674).
struct Layout {
  Shape shape_;
  std::vector<size_t> strides_;
  size_t offset_ = 0;

  static Layout from_shape(const Shape& s) {
    Layout l;
    l.shape_ = s;
    l.strides_ = s.stride_contiguous();
    return l;
  }
  const Shape& shape() const { return shape_; }
  const std::vector<size_t>& dims() const { return shape_.dims(); }
  const std::vector<size_t>& strides() const { return strides_; }
  size_t rank() const { return shape_.rank(); }
  size_t offset() const { return offset_; }
  void set_offset(size_t o) { offset_ = o; }
  size_t num_elements() const { return shape_.num_elements(); }

  // layout.rs:585-597: rank <= 1 is never "compressible".
  bool can_be_compressed() const {
    const auto& d = dims();
    if (d.size() <= 1) return false;
    for (size_t i = 0; i + 1 < d.size(); ++i)
      if (strides_[i] != strides_[i + 1] * d[i + 1]) return false;
    return true;
  }
  // layout.rs:599-610
  Layout compress_all() const {
    const auto& d = dims();
    for (size_t i = 0; i + 1 < d.size(); ++i)
      if (strides_[i] != strides_[i + 1] * d[i + 1]) bail("cannot collapse dims");
    Layout l;
    l.shape_ = Shape({num_elements()});
    l.strides_ = {strides_.empty() ? 1 : strides_.back()};
    l.offset_ = offset_;
    return l;
  }
  // layout.rs:624-634: swap the last two dims.
  Layout transpose() const {
    size_t r = rank();
    if (r < 2) return *this;
    Layout l = *this;
    std::swap(l.shape_.dims_[r - 2], l.shape_.dims_[r - 1]);
    std::swap(l.strides_[r - 2], l.strides_[r - 1]);
    return l;
  }
  bool operator==(const Layout& o) const { return shape_ == o.shape_ && strides_ == o.strides_ && offset_ == o.offset_; }
  std::string key() const {
    std::string s = "L";
    for (size_t d : dims()) s += std::to_string(d) + ",";
    s += "/";
    for (size_t d : strides_) s += std::to_string(d) + ",";
    return s + "+" + std::to_string(offset_);
  }
};

// lang.rs:5-32
enum class ReduceOp : int { Sum = UGHIP_R_SUM, Max = UGHIP_R_MAX, Min = UGHIP_R_MIN };
enum class UnaryOp : int { Id = UGHIP_U_ID, Exp = UGHIP_U_EXP, Sin = UGHIP_U_SIN, Cos = UGHIP_U_COS, Neg = UGHIP_U_NEG, Sqrt = UGHIP_U_SQRT, Cast = UGHIP_U_CAST };
enum class BinaryOp : int { Add = UGHIP_B_ADD, Sub = UGHIP_B_SUB, Mul = UGHIP_B_MUL, Div = UGHIP_B_DIV, Mod = UGHIP_B_MOD, Min = UGHIP_B_MIN, Max = UGHIP_B_MAX };

// lang.rs:34-45
struct LaunchConfig {
  uint32_t grid_dim = 1, block_dim = 1, shared_mem = 0;
  static LaunchConfig for_num_elems(uint32_t n) { return {(n + 31) / 32, 32, 0}; }
};

}  // namespace ug
