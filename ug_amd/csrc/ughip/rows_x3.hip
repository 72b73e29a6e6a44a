// 33 .. 128 f32 rows against a bf16 matrix [n, k] as three bf16 terms per row element, on the bf16 matrix pipe, with the split done
// inside the product: x [m, k] f32 is read as it is, no planes go through memory.
//
//   unit      = one k tile (64) of one column tile (128 columns): 128 x 128 x 64 x 3 terms, 96 MFMAs of 16 x 16 x 32 per wave
//   workgroup = 8 waves, takes `units` consecutive units of the (column tile, k tile) order -- a stream-K split: with 11264
//               columns and k = 2048 that is 2816 units, 11 for each of 256 workgroups, where whole tiles would leave 80 CUs idle
//               (88 tiles x 2) or need a second round (88 x 3).  A workgroup whose units cross into the next column tile stores one
//               slab of partial sums per tile it touches; slab s of a tile is the s-th workgroup that touches it, and the fold
//               adds them in that order, so the result does not depend on timing.
//   waves 0-3 : the products.  Wave w owns rows 32 w .. 32 w + 31 and all 128 columns: 16 accumulators.  The matrix tile's
//               fragments (16 x 128 bits) are read from LDS once per unit and meet the three planes in turn; the row fragments
//               come from LDS plane by plane.  These waves also send the matrix tiles on their way: global -> LDS
//               (global_load_lds_dwordx4), three units ahead in a ring of four stages, four instructions per wave and unit.
//   waves 4-7 : the rows.  Each loads its part of the 128 x 64 f32 tile of the next unit but one (16-byte loads, rows 256 bytes
//               apart in memory: whole lines), splits every element into hi + mid + lo (v_cvt_pk_bf16_f32 rounds to nearest
//               even; the remainders are exact) and writes the three planes into one of two LDS stages in the layout the
//               fragment reads want.  Their VALU work shares the SIMDs with the MFMAs of waves 0-3, which leave the issue
//               port idle three cycles in four.
//   barrier t : in front of the last plane of unit t - 1.  Says that tile t and planes t are in LDS and that nobody reads the LDS
//               of unit t - 1 any more (its fragments are in registers by then); the last plane of unit t - 1 then runs while the
//               fragments of unit t arrive, so the matrix pipe does not wait behind the barrier.
//   LDS       : 4 x 16 KiB matrix stages + 2 x 48 KiB plane stages = 160 KiB, one workgroup per CU.
//
// What bounds it: the matrix pipe at the rate the power limit allows with random operands (1.7-1.8 PFLOP/s: 0.96 us per unit with
// every CU busy), plus 4 us of launch, first tile and slab stores; barriers and LDS traffic add a quarter, the conversions and
// the rows' loads (32 KiB per unit and CU from L2, where planes written by a kernel in front would be 48) a tenth each.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <type_traits>

#include "gemm.h"
#include "internal.h"
#include "ughip.h"

namespace ughip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x4 mma16(const u32x4& a, const u32x4& b, const f32x4& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }
// Every lane's 16 bytes at base + voff go to LDS at lds_byte_addr + lane * 16.  The compiler does not see the load: the waits are explicit.
__device__ __forceinline__ void dma16(const void* base, unsigned voff, unsigned lds_byte_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_byte_addr), "v"(voff), "s"(base) : "memory", "m0");
}
// k-contiguous tile ([rows][64] bf16): 128-byte rows of 8 chunks of 16 bytes, chunk' = chunk ^ ((row / 2) & 7): the fragment reads
// (16 rows x 4 chunks per instruction) then meet every bank once
__device__ __forceinline__ int kc_idx(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }

constexpr int BN = 128, BM = 128;
constexpr int NB = 4;  // stages of the matrix ring
constexpr int B_STAGE = BN * 64 * 2, B_BYTES = NB * B_STAGE, PLANE = BM * 64 * 2, A_STAGE = 3 * PLANE, LDS_TOTAL = B_BYTES + 2 * A_STAGE;

// x = hi + mid + lo, every term a bf16 (round to nearest even of what the terms before left: the remainders are exact, so
// |x - (hi + mid + lo)| <= 2^-25 |x|).  An infinity (given, or reached when |x| rounds up past the largest bf16) is all in hi: its
// remainders would be inf - inf, and the product has to give what the f32 pipe gives for such an x.  A NaN is all in hi as well
// where the code that looks for infinities runs, and three NaNs where it does not: a NaN either way.
template <bool FINITE>
__device__ __forceinline__ void split_pair(float x0, float x1, unsigned& hi, unsigned& mid, unsigned& lo) {
  const unsigned h = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{x0, x1}, bf16x2));
  float r0 = x0 - __uint_as_float(h << 16), r1 = x1 - __uint_as_float(h & 0xffff0000u);
  if (!FINITE) {
    if ((h & 0x7f80u) == 0x7f80u) r0 = 0.f;
    if ((h & 0x7f800000u) == 0x7f800000u) r1 = 0.f;
  }
  const unsigned m = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{r0, r1}, bf16x2));
  const float q0 = r0 - __uint_as_float(m << 16), q1 = r1 - __uint_as_float(m & 0xffff0000u);
  hi = h, mid = m, lo = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{q0, q1}, bf16x2));
}

// x: [m][k] f32, m <= 128; w: [n][k] bf16; slabs: [S][m][n] f32.  Unit u = T * KT + kt (T: column tile, kt: k tile);
// workgroup g takes units [g U, min(g U + U, total)) and writes slab g - (T KT) / U of every tile T it touches.
__global__ void __launch_bounds__(512) rows_x3_kernel(const float* __restrict__ x, const uint16_t* __restrict__ w, float* __restrict__ slabs, int m, int n, int k, int KT,
                                                      int U, int total) {
  extern __shared__ u32x4 lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int u0 = blockIdx.x * U, nU = min(U, total - u0);
  if (wave >= 4) {
    // 32 instructions of 64 lanes x 4 floats cover the 128 x 64 tile; this wave takes instructions c, c + 4, ...
    const int c = wave - 4;
    constexpr int NQ = 8;
    f32x4 raw[2][NQ];
    unsigned goff[NQ];  // byte offset of the lane's 4 floats inside x, without the k tile (rows past the end read the last row: not stored)
    unsigned loff[NQ];  // byte offset inside a plane of the stage
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
      const int q = c + 4 * i, e = q * 64 + lane, row = e >> 4, kq = e & 15;
      goff[i] = (unsigned)min(row, m - 1) * (unsigned)k * 4u + kq * 16;
      loff[i] = (unsigned)(kc_idx(row, kq >> 1) * 16 + (kq & 1) * 8);
    }
    auto load = [&](int set, int t) __attribute__((always_inline)) {
      const int kt = (u0 + min(t, nU - 1)) % KT;  // past the last unit: the last one again, unused
      const char* base = reinterpret_cast<const char*>(x) + (size_t)kt * 256;
#pragma unroll
      for (int i = 0; i < NQ; ++i) raw[set][i] = *reinterpret_cast<const f32x4*>(base + goff[i]);
    };
    auto convert = [&](int set, int t) __attribute__((always_inline)) {
      char __attribute__((address_space(3)))* dst = (char __attribute__((address_space(3)))*)lds + B_BYTES + (t & 1) * A_STAGE;
      // an element that is, or rounds to, an infinity is rare: one test for the wave's 2048 elements chooses the code that looks for them
      float big = 0.f;
#pragma unroll
      for (int i = 0; i < NQ; ++i) big = fmaxf(big, fmaxf(fmaxf(fabsf(raw[set][i][0]), fabsf(raw[set][i][1])), fmaxf(fabsf(raw[set][i][2]), fabsf(raw[set][i][3]))));
#define UGHIP_ROWS_X3_CONVERT(FIN)                                                          \
  _Pragma("unroll") for (int i = 0; i < NQ; ++i) {                                          \
    unsigned h0, m0, l0, h1, m1, l1;                                                        \
    const f32x4 v = raw[set][i];                                                            \
    split_pair<FIN>(v[0], v[1], h0, m0, l0);                                                \
    split_pair<FIN>(v[2], v[3], h1, m1, l1);                                                \
    *(u32x2 __attribute__((address_space(3)))*)(dst + loff[i]) = u32x2{h0, h1};             \
    *(u32x2 __attribute__((address_space(3)))*)(dst + PLANE + loff[i]) = u32x2{m0, m1};     \
    *(u32x2 __attribute__((address_space(3)))*)(dst + 2 * PLANE + loff[i]) = u32x2{l0, l1}; \
  }
      if (__builtin_amdgcn_ballot_w64(big >= __uint_as_float(0x7f7f8000u)) != 0) {  // 0x7f7f8000 and up round to the bf16 infinity
        UGHIP_ROWS_X3_CONVERT(false)
      } else {
        UGHIP_ROWS_X3_CONVERT(true)
      }
#undef UGHIP_ROWS_X3_CONVERT
    };
    load(0, 0);
    load(1, 1);
    convert(0, 0);
    wait_lgkmcnt0();  // the planes are in LDS
    __builtin_amdgcn_s_barrier();  // barrier 0
    for (int t = 1; t < nU; t += 2) {
      load(0, t + 1);
      convert(1, t);
      wait_lgkmcnt0();
      __builtin_amdgcn_s_barrier();  // barrier t
      if (t + 1 < nU) {
        load(1, t + 2);
        convert(0, t + 1);
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();  // barrier t + 1
      }
    }
    return;
  }
  const unsigned lds_addr = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds;
  auto issue = [&](int t) {
    const int u = u0 + t, T = u / KT, kt = u - T * KT;
    const int n_left = n - T * BN;  // a last tile may hang over the end of n: rows past the end fetch the last row again, their columns are not stored
    const char* base = reinterpret_cast<const char*>(w) + ((size_t)T * BN * k + (size_t)kt * 64) * 2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = wave + 4 * i, row = q * 8 + (lane >> 3), cp = lane & 7;
      const unsigned vo = (unsigned)(min(row, n_left - 1) * k * 2 + ((cp ^ ((row >> 1) & 7)) << 4));
      dma16(base, vo, lds_addr + (t % NB) * B_STAGE + q * 1024);
    }
  };
  int issued = 0;
  // This wave's part of tile t has landed: loads return in order, so with `ahead` younger tiles on their way at most 4 * ahead
  // loads may be outstanding.  (The slab stores of a tile boundary retire in no fixed order against loads, but they can only add
  // to the count: a tile that has not landed keeps every younger load outstanding as well.)
  auto wait_tile = [&](int t) {
    const int ahead = issued - 1 - t;
    if (ahead >= 2) wait_vmcnt<8>();
    else if (ahead == 1) wait_vmcnt<4>();
    else wait_vmcnt<0>();
  };
  const int r_base = wave * 32;
  u32x4 fa[2][2][2], bf[2][8];
  f32x4 acc[2][8];
  auto zero = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  };
  zero();
  // lane l feeds row / column l % 16, k = 8 (l / 16) .. + 7 of a step of 32
  auto read_a = [&](int set, int t, int p) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int s = 0; s < 2; ++s) fa[set][i][s] = lds[(B_BYTES + (t & 1) * A_STAGE + p * PLANE) / 16 + kc_idx(r_base + 16 * i + (lane & 15), 4 * s + (lane >> 4))];
  };
  auto read_b = [&](int t, int s, int j) { bf[s][j] = lds[(t % NB) * (B_STAGE / 16) + kc_idx(16 * j + (lane & 15), 4 * s + (lane >> 4))]; };
  auto plane = [&](int set) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i) acc[i][j] = mma16(bf[s][j], fa[set][i][s], acc[i][j]);  // operands swapped: a lane holds 4 consecutive columns of one row
  };
  // Register e of lane l of block (i, j): row r_base + 16 i + l % 16, column 16 j + 4 (l / 16) + e.
  auto finish = [&](int t) {
    const int u = u0 + t, T = u / KT;
    if (t + 1 >= nU || (u + 1) / KT != T) {
      const int slab = blockIdx.x - (T * KT) / U;
      float* out = slabs + (size_t)slab * m * n + (size_t)T * BN;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int row = r_base + 16 * i + (lane & 15), col = 16 * j + (lane >> 4) * 4;
          if (row < m && T * BN + col < n) *reinterpret_cast<f32x4*>(out + (size_t)row * n + col) = acc[i][j];  // n % 8 == 0: 4 columns exist whole or not at all
        }
      zero();
    }
  };
  for (; issued < min(nU, NB - 1); ++issued) issue(issued);
  wait_tile(0);
  __builtin_amdgcn_s_barrier();  // barrier 0
  if (issued < nU) {
    issue(issued);
    ++issued;
  }
  read_a(0, 0, 0);
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < 8; ++j) read_b(0, s, j);
  // P: the register set of the unit's first plane (sets alternate plane by plane, and a unit has three)
  auto unit = [&](int t, auto par) {
    constexpr int P = decltype(par)::value;
    const bool more = t + 1 < nU;
    read_a(P ^ 1, t, 1);
    plane(P);
    read_a(P, t, 2);
    plane(P ^ 1);
    if (more) {
      wait_tile(t + 1);
      wait_lgkmcnt0();  // this unit's last fragments are in registers: its LDS may be written again behind the barrier
      __builtin_amdgcn_s_barrier();  // barrier t + 1
      if (issued < nU) {  // into the stage of tile t - 1, whose fragments were read in front of barrier t
        issue(issued);
        ++issued;
      }
      read_a(P ^ 1, t + 1, 0);
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < 2; ++i) acc[i][j] = mma16(bf[s][j], fa[P][i][s], acc[i][j]);
        if (more) read_b(t + 1, s, j);  // behind the last use of this unit's fragment
      }
    finish(t);
  };
  for (int t = 0; t < nU; t += 2) {
    unit(t, std::integral_constant<int, 0>());
    if (t + 1 < nU) unit(t + 1, std::integral_constant<int, 1>());
  }
}

// c = the slabs of every column tile added in slab order, then the epilogue: NONE, ADD (+ residual[m, n]) or SWIGLU
// (c[m, n / 2] = silu(sum[:, :n / 2]) * sum[:, n / 2:], x / (1 + exp(-x)) as the lazy graph of ug-llama/src/model.rs:44-52 computes it).
// Tile T has the slabs of the workgroups (T KT) / U .. (T KT + KT - 1) / U.
__device__ __forceinline__ f32x4 tile_sum(const float* __restrict__ slabs, size_t slab_elems, size_t at, int col, int KT, int U) {
  const int T = col / BN, first = (T * KT) / U, last = (T * KT + KT - 1) / U, cnt = last - first;
  f32x4 s = *reinterpret_cast<const f32x4*>(slabs + at);
  // eight slabs at a time, all eight loads on their way before the first is added (a slab past the last is the last one again,
  // loaded and not added): the order of the sum stays slab by slab
  for (int g = 1; g <= cnt; g += 8) {
    f32x4 v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = *reinterpret_cast<const f32x4*>(slabs + (size_t)min(g + e, cnt) * slab_elems + at);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (g + e <= cnt) s += v[e];
  }
  return s;
}
template <int EPI>
__global__ void __launch_bounds__(256) rows_x3_fold(const float* __restrict__ slabs, float* __restrict__ c, const float* __restrict__ residual, int m, int n, int KT, int U) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t slab_elems = (size_t)m * n;
  if constexpr (EPI == GemmEpilogue::SWIGLU) {
    const size_t half4 = (size_t)n / 8;
    if (g >= (size_t)m * half4) return;
    const size_t r = g / half4, j4 = g % half4;
    const int col = (int)(j4 * 4);
    const f32x4 a = tile_sum(slabs, slab_elems, r * n + col, col, KT, U), b = tile_sum(slabs, slab_elems, r * n + n / 2 + col, n / 2 + col, KT, U);
    f32x4 s;
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] = a[e] / (1.f + expf(-a[e])) * b[e];
    *reinterpret_cast<f32x4*>(c + g * 4) = s;
  } else {
    if (g >= slab_elems / 4) return;
    const int col = (int)((g * 4) % (size_t)n);
    f32x4 s = tile_sum(slabs, slab_elems, g * 4, col, KT, U);
    if constexpr (EPI == GemmEpilogue::ADD) s += *reinterpret_cast<const f32x4*>(residual + g * 4);
    *reinterpret_cast<f32x4*>(c + g * 4) = s;
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

bool rows_x3_supported(const void* x, const void* w, const void* c, const void* residual, size_t m, size_t n, size_t k) {
  // (the unit count and the byte offsets inside one column tile's rows are held in 32 bits)
  return m >= 1 && m <= (size_t)BM && n >= 8 && n % 8 == 0 && k >= 64 && k % 64 == 0 && k <= (1u << 20) && n <= (1u << 24) && n * k <= (1ull << 31) && aligned16(x) &&
         aligned16(w) && aligned16(c) && aligned16(residual);
}

// Units per workgroup: every CU busy in one round, and past that as few slabs as the units' time allows -- a unit costs a
// microsecond of a workgroup's time, a slab (64 KiB written, read once by the fold) about half a microsecond of everybody's.
RowsX3Plan rows_x3_plan(size_t m, size_t n, size_t k, int forced_units, int num_cus) {
  RowsX3Plan pl;
  const int KT = (int)(k / 64), tiles = (int)((n + BN - 1) / BN), total = tiles * KT;
  const int cus = num_cus > 0 ? num_cus : 256;
  auto fill = [&](int U, RowsX3Plan* out) {
    out->units = U, out->groups = (total + U - 1) / U, out->max_slabs = 0;
    int segments = 0;
    for (int g = 0; g < out->groups; ++g) segments += (std::min(g * U + U, total) - 1) / KT - (g * U) / KT + 1;
    for (int T = 0; T < tiles; ++T) out->max_slabs = std::max(out->max_slabs, (T * KT + KT - 1) / U - (T * KT) / U + 1);
    return (double)U + segments * 65536.0 / 1e6 / 2.0;
  };
  const int u_min = (total + cus - 1) / cus;
  if (forced_units > 0) {
    fill(std::max(forced_units, u_min), &pl);
  } else {
    double best = 0;
    for (int U = u_min; U <= std::max(u_min, KT); ++U) {
      RowsX3Plan cand;
      const double cost = fill(U, &cand);
      if (cand.max_slabs > 16) continue;
      if (pl.units == 0 || cost < best) pl = cand, best = cost;
    }
    if (pl.units == 0) fill(std::max(u_min, KT), &pl);
  }
  pl.ws_bytes = (size_t)pl.max_slabs * m * n * sizeof(float);
  return pl;
}

void rows_x3_name(const RowsX3Plan& pl, GemmEpilogue::Kind kind, char* out, size_t out_len) {
  snprintf(out, out_len, "rows_x3<128x128,3 terms split in the kernel,%d units x %d workgroups,%d slabs%s>", pl.units, pl.groups, pl.max_slabs,
           kind == GemmEpilogue::SWIGLU ? ",swiglu fold" : kind == GemmEpilogue::ADD ? ",+residual in the fold" : pl.max_slabs == 1 ? ",no fold" : ",fold");
}

hipError_t rows_x3_launch(hipStream_t stream, const float* x, const void* w, float* ws, float* c, size_t m, size_t n, size_t k, const RowsX3Plan& pl, GemmEpilogue::Kind kind,
                          const float* residual) {
  static std::atomic<unsigned long long> configured{0};  // one bit per device: the attribute is per device
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
  if (!bit || !(configured.load(std::memory_order_relaxed) & bit)) {
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(rows_x3_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_TOTAL)) return e;
    configured.fetch_or(bit, std::memory_order_relaxed);
  }
  const int KT = (int)(k / 64), tiles = (int)((n + BN - 1) / BN), total = tiles * KT;
  // one slab per tile and nothing for the fold to do: the slab is the result
  const bool direct = pl.max_slabs == 1 && kind == GemmEpilogue::NONE;
  rows_x3_kernel<<<dim3((unsigned)pl.groups), dim3(512), LDS_TOTAL, stream>>>(x, static_cast<const uint16_t*>(w), direct ? c : ws, (int)m, (int)n, (int)k, KT, pl.units, total);
  if (hipError_t e = hipGetLastError()) return e;
  if (direct) {
    char name[160];
    rows_x3_name(pl, kind, name, sizeof name);
    note_kernel("%s", name);
    return hipSuccess;
  }
  const size_t groups4 = kind == GemmEpilogue::SWIGLU ? m * n / 8 : m * n / 4;
  const dim3 grid((unsigned)((groups4 + 255) / 256));
  if (kind == GemmEpilogue::ADD)
    rows_x3_fold<GemmEpilogue::ADD><<<grid, dim3(256), 0, stream>>>(ws, c, residual, (int)m, (int)n, KT, pl.units);
  else if (kind == GemmEpilogue::SWIGLU)
    rows_x3_fold<GemmEpilogue::SWIGLU><<<grid, dim3(256), 0, stream>>>(ws, c, nullptr, (int)m, (int)n, KT, pl.units);
  else
    rows_x3_fold<GemmEpilogue::NONE><<<grid, dim3(256), 0, stream>>>(ws, c, nullptr, (int)m, (int)n, KT, pl.units);
  char name[160];
  rows_x3_name(pl, kind, name, sizeof name);
  note_kernel("%s", name);
  return hipGetLastError();
}

}  // namespace ughip
