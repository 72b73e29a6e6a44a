// Element type conversion on the device: dst[i] = (dst dtype) src[i] for the five dtypes of
// ug-core/src/dtype.rs:5-12.  This is the loop ug-core/src/safetensors.rs:141-271 runs on the host
// before every upload (load_with_cast), moved behind the upload: a bf16 checkpoint crosses the
// host link as 2 bytes per weight and is widened in HBM.
//
// Numerics follow that host code: 16-bit floats widen exactly; f32 -> bf16/f16 rounds to nearest
// even (half::{bf16,f16}::from_f32); float -> integer truncates toward zero, saturates, and maps
// NaN to 0 (Rust `as`); integers reach the 16-bit floats through f32; i64 -> i32 wraps.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

#include "internal.h"
#include "ughip.h"

using namespace ughip;

namespace {

template <int DT>
struct Elem;
template <>
struct Elem<UGHIP_BF16> {
  typedef uint16_t type;
};
template <>
struct Elem<UGHIP_F16> {
  typedef uint16_t type;
};
template <>
struct Elem<UGHIP_F32> {
  typedef float type;
};
template <>
struct Elem<UGHIP_I32> {
  typedef int32_t type;
};
template <>
struct Elem<UGHIP_I64> {
  typedef int64_t type;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
// half::bf16::from_f32: NaN keeps its sign and becomes quiet; everything else rounds to nearest even.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  const uint32_t x = __float_as_uint(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
  const uint32_t round_bit = 0x8000u;
  if ((x & round_bit) != 0 && (x & (3 * round_bit - 1)) != 0) return (uint16_t)((x >> 16) + 1);
  return (uint16_t)(x >> 16);
}
__device__ __forceinline__ float f16_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ uint16_t f32_to_f16(float f) { return __half_as_ushort(__float2half_rn(f)); }

// Rust `f32 as i32` / `as i64`.
__device__ __forceinline__ int32_t f32_to_i32(float f) {
  if (f != f) return 0;
  if (f >= 2147483648.f) return INT32_MAX;
  if (f <= -2147483648.f) return INT32_MIN;
  return (int32_t)f;
}
__device__ __forceinline__ int64_t f32_to_i64(float f) {
  if (f != f) return 0;
  if (f >= 9223372036854775808.f) return INT64_MAX;
  if (f <= -9223372036854775808.f) return INT64_MIN;
  return (int64_t)f;
}

template <int S>
__device__ __forceinline__ float to_f32(typename Elem<S>::type v) {
  if (S == UGHIP_BF16) return bf16_to_f32((uint16_t)v);
  if (S == UGHIP_F16) return f16_to_f32((uint16_t)v);
  return (float)v;  // f32, i32, i64 (`as f32`: round to nearest even)
}

template <int S, int D>
__device__ __forceinline__ typename Elem<D>::type convert_one(typename Elem<S>::type v) {
  if (S == D) return (typename Elem<D>::type)v;
  if (S == UGHIP_I32 && D == UGHIP_I64) return (typename Elem<D>::type)(int64_t)(int32_t)v;
  if (S == UGHIP_I64 && D == UGHIP_I32) return (typename Elem<D>::type)(int32_t)(int64_t)v;  // wraps
  const float f = to_f32<S>(v);
  if (D == UGHIP_BF16) return (typename Elem<D>::type)f32_to_bf16(f);
  if (D == UGHIP_F16) return (typename Elem<D>::type)f32_to_f16(f);
  if (D == UGHIP_F32) return (typename Elem<D>::type)f;
  if (D == UGHIP_I32) return (typename Elem<D>::type)f32_to_i32(f);
  return (typename Elem<D>::type)f32_to_i64(f);
}

// Four consecutive elements per thread: the wider side moves 16 (or 32) bytes per lane.
template <int S, int D>
__global__ void __launch_bounds__(256) convert_kernel(const typename Elem<S>::type* __restrict__ src, typename Elem<D>::type* __restrict__ dst, size_t n) {
  typedef typename Elem<S>::type ST;
  typedef typename Elem<D>::type DT;
  typedef ST SV __attribute__((ext_vector_type(4)));
  typedef DT DV __attribute__((ext_vector_type(4)));
  const size_t g = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (g + 4 <= n) {
    const SV s = __builtin_nontemporal_load(reinterpret_cast<const SV*>(src + g));  // read once: no cache line claimed (2^27 bf16 -> f32: 130 -> 126 us on one box)
    DV d;
    d.x = convert_one<S, D>(s.x);
    d.y = convert_one<S, D>(s.y);
    d.z = convert_one<S, D>(s.z);
    d.w = convert_one<S, D>(s.w);
    *reinterpret_cast<DV*>(dst + g) = d;
  } else {
    for (size_t i = g; i < n; ++i) dst[i] = convert_one<S, D>(src[i]);
  }
}

template <int S, int D>
void launch(hipStream_t st, const void* src, void* dst, size_t n) {
  const size_t threads = (n + 3) / 4;
  convert_kernel<S, D><<<(unsigned)((threads + 255) / 256), 256, 0, st>>>(static_cast<const typename Elem<S>::type*>(src),
                                                                        static_cast<typename Elem<D>::type*>(dst), n);
}

template <int S>
void launch_from(hipStream_t st, int d, const void* src, void* dst, size_t n) {
  switch (d) {
    case UGHIP_BF16: return launch<S, UGHIP_BF16>(st, src, dst, n);
    case UGHIP_F16: return launch<S, UGHIP_F16>(st, src, dst, n);
    case UGHIP_F32: return launch<S, UGHIP_F32>(st, src, dst, n);
    case UGHIP_I32: return launch<S, UGHIP_I32>(st, src, dst, n);
    default: return launch<S, UGHIP_I64>(st, src, dst, n);
  }
}

}  // namespace

extern "C" int ughip_convert(ughip_device* dev, const ughip_slice* src, ughip_slice* dst) {
  if (!dev || !src || !dst) return set_error(UGHIP_ERR_INVALID, "convert: null device or slice");
  if (src->len != dst->len) return set_error(UGHIP_ERR_INVALID, "convert: src has %zu elements, dst %zu", src->len, dst->len);
  if (src == dst) return set_error(UGHIP_ERR_INVALID, "convert: src and dst alias");
  if (src->dev != dev || dst->dev != dev) return set_error(UGHIP_ERR_INVALID, "convert: slice lives on another device");
  const size_t n = src->len;
  if (n == 0) return UGHIP_OK;
  if (n > (size_t)0x7fffffff * 1024) return set_error(UGHIP_ERR_INVALID, "convert: %zu elements exceed one launch", n);
  if (int rc = device_activate(dev)) return rc;
  switch (src->dtype) {
    case UGHIP_BF16: launch_from<UGHIP_BF16>(dev->stream, dst->dtype, src->ptr, dst->ptr, n); break;
    case UGHIP_F16: launch_from<UGHIP_F16>(dev->stream, dst->dtype, src->ptr, dst->ptr, n); break;
    case UGHIP_F32: launch_from<UGHIP_F32>(dev->stream, dst->dtype, src->ptr, dst->ptr, n); break;
    case UGHIP_I32: launch_from<UGHIP_I32>(dev->stream, dst->dtype, src->ptr, dst->ptr, n); break;
    case UGHIP_I64: launch_from<UGHIP_I64>(dev->stream, dst->dtype, src->ptr, dst->ptr, n); break;
    default: return set_error(UGHIP_ERR_INVALID, "convert: unknown dtype %d", src->dtype);
  }
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}
