// Reductions over the 64 lanes of a wavefront, shared by the hand-written kernels.
//
// Both are butterflies with partners at distance 32, 16, 8, 4, 2, 1 in that order: every lane ends
// with the same value, and a sum has the same association tree wherever it is computed, so kernels
// that fold the same numbers in the same lane layout agree to the bit.  After the step at
// distance d, lanes that differ only in bit d hold equal values; the last four steps therefore take
// a rotation within rows of 16 lanes (lane i reads lane (i + d) mod 16 of its row, a
// register-to-register DPP move) in place of an exchange through the LDS crossbar: (i + d) mod 16
// differs from i ^ d only in bits already folded.
#pragma once
#include <hip/hip_runtime.h>

namespace ughip {

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
constexpr int DPP_ROW_ROR8 = 0x128, DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR2 = 0x122, DPP_ROW_ROR1 = 0x121;

// The steps at distance 8, 4, 2, 1 of a sum butterfly whose earlier steps (if any) have run.
__device__ __forceinline__ float row_sum16(float v) {
  v += dpp_move<DPP_ROW_ROR8>(v);
  v += dpp_move<DPP_ROW_ROR4>(v);
  v += dpp_move<DPP_ROW_ROR2>(v);
  v += dpp_move<DPP_ROW_ROR1>(v);
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
  v += __shfl_xor(v, 32, 64);
  v += __shfl_xor(v, 16, 64);
  return row_sum16(v);
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, dpp_move<DPP_ROW_ROR8>(v));
  v = fmaxf(v, dpp_move<DPP_ROW_ROR4>(v));
  v = fmaxf(v, dpp_move<DPP_ROW_ROR2>(v));
  v = fmaxf(v, dpp_move<DPP_ROW_ROR1>(v));
  return v;
}

}  // namespace ughip
