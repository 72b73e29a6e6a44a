// Three bf16 terms of an f32 value and where they live in memory: shared by the kernels that write such planes.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace ughip {

// x = hi + mid + lo with every term a bf16 (round to nearest even of what the terms before left): 24 mantissa bits in
// three pieces, so |x - (hi + mid + lo)| <= 2^-25 |x|.  x3 row r holds, for every 64 columns c0 .. c0 + 63 of x, the
// three planes side by side: [hi(c0..) | mid(c0..) | lo(c0..)], i.e. K tile t of x3 is plane t % 3 of K tile t / 3 of x,
// and the three of them meet the same K tile of the matrix one after the other.
__device__ __forceinline__ uint16_t bf16_rne(float f) {
  const uint32_t x = __float_as_uint(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);  // NaN stays NaN
  return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}
// hi + mid + lo of one value
__device__ __forceinline__ void split3(float x, uint16_t& hi, uint16_t& mid, uint16_t& lo) {
  hi = bf16_rne(x);
  const float h = __uint_as_float((uint32_t)hi << 16);
  // an infinity (given, or reached when |x| rounds up past the largest bf16) or a NaN is all in the first term: the
  // remainders would be inf - inf, and the product has to give what the f32 pipe gives for such an x
  const bool fin = (hi & 0x7f80) != 0x7f80;
  const float r1 = fin ? x - h : 0.f;  // exact: hi shares the leading bits of x
  mid = bf16_rne(r1);
  const float r2 = r1 - __uint_as_float((uint32_t)mid << 16);
  lo = bf16_rne(r2);
}

// Four consecutive elements of a row of k, split, to their places in the row's planes (x3_row: the row's first element).
__device__ __forceinline__ void split3_store4(const float in[4], uint16_t* __restrict__ x3_row, size_t col) {
  uint16_t hi[4], mid[4], lo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) split3(in[i], hi[i], mid[i], lo[i]);
  uint16_t* o = x3_row + (col / 64) * 192 + col % 64;
  *reinterpret_cast<ushort4*>(o) = make_ushort4(hi[0], hi[1], hi[2], hi[3]);
  *reinterpret_cast<ushort4*>(o + 64) = make_ushort4(mid[0], mid[1], mid[2], mid[3]);
  *reinterpret_cast<ushort4*>(o + 128) = make_ushort4(lo[0], lo[1], lo[2], lo[3]);
}

}  // namespace ughip
