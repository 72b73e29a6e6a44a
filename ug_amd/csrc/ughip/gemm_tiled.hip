// Tuned MFMA GEMM for gfx950: C[b] = A[b] x B[b], f32 accumulate.
//
//   block tile BM x BN: 256x128 with 8 waves (4 x 2, two per SIMD), 128x128 or 128x64 with 4 waves
//   (2 x 2); each wave owns a block of MFMA 32x32 accumulators
//   K tile = 128 bytes per matrix row (64 bf16 / 32 f32), double-buffered in LDS; global loads run
//   two tiles ahead through two register sets, LDS staging stores and fragment reads are spread
//   between the MFMAs of the tile being multiplied
//   LDS rows are 8 chunks of 16 bytes, chunk' = chunk ^ ((row / 2) & 7): every 128-bit fragment read
//   and every staging write is bank-conflict free on the 64-bank LDS
//   a row-major B ([k, n]) is transposed in registers on its way to LDS so that both MFMA
//   operands read 128 bits of consecutive k (v_perm_b32 for bf16; free for f32)
//   tiles are handed to workgroups XCD by XCD so that the tiles of one batch element share an L2
//   16-bit products whose 256 x 256 or 256 x 128 tiles fill the chip go to gemm_dma.hip instead (matmul.hip decides)
//
// bf16, f16: v_mfma_f32_32x32x16_{bf16,f16} (lane l feeds row/col l%32, k = 8*(l/32)..+7).
// f32:  v_mfma_f32_32x32x2_f32   (lane l feeds row/col l%32, k = l/32); the 4 floats of a 128-bit
//       fragment feed 4 consecutive MFMAs, lanes 0-31 holding k..k+3 and lanes 32-63 k+4..k+7.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "gemm.h"
#include "internal.h"
#include "ughip.h"

namespace ughip {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
// native vectors, not HIP's uint4/uint2 structs: copies of those become memcpy calls that keep the
// prefetch registers in scratch memory
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int CHUNKS = 8;  // 16-byte chunks per 128-byte LDS row

template <typename T>
struct Elt;
template <>
struct Elt<float> {
  static constexpr int BK = 32, VE = 4;
};
template <>
struct Elt<__bf16> {
  static constexpr int BK = 64, VE = 8;
};
template <>
struct Elt<_Float16> {
  static constexpr int BK = 64, VE = 8;
};

// One 32x32x16 MFMA on 8 consecutive k of a 16-bit type.
__device__ __forceinline__ floatx16 mma16(__bf16, const u32x4& a, const u32x4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mma16(_Float16, const u32x4& a, const u32x4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mma16(float, const u32x4&, const u32x4&, const floatx16& c) { return c; }  // never taken

// 64 banks x 4 bytes: two 128-byte rows span the banks once, so the chunk is rotated by row / 2 --
// 16 lanes reading one chunk column of 16 consecutive rows then touch 16 different bank groups.
__device__ __forceinline__ int lds_swz(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int lds_idx(int row, int chunk) { return row * CHUNKS + (chunk ^ lds_swz(row)); }

// The tile being prefetched from global memory while the previous one is multiplied.
template <int BM, int NT>
struct Staged {
  u32x4 a[BM * 8 / NT];  // NT threads move NT / 8 rows of 8 chunks per pass
  u32x4 b[4];
};

// B_NK: 0 = rhs [k, n] row-major, 1 = rhs [n, k] row-major, 2 = [n, k] row-major stored as bf16 under an
// f32 product (BT = uint16_t): a chunk of 4 elements is 8 bytes in memory and is widened on its way
// into LDS (exact), so the product is bit for bit the f32 one on the widened values.
template <typename T, int B_NK>
struct RhsElt {
  typedef T type;
};
template <>
struct RhsElt<float, 2> {
  typedef uint16_t type;
};

__device__ __forceinline__ u32x4 widen_bf16x4(const u32x4& r) { return u32x4{r.x << 16, r.x & 0xffff0000u, r.y << 16, r.y & 0xffff0000u}; }

// RAGGED: the tile may hang over the last row of the lhs or (B_NK != 0) of the rhs; p.M and p.n_tile are then
// the rows and columns of THIS tile that exist, and rows past them read the last one (their products are
// never stored).
template <typename T, int B_NK, int BM, int BN, int NT, bool RAGGED = false, typename BT>
__device__ __forceinline__ void load_tiles(const T* __restrict__ A, const BT* __restrict__ B, const MMArgs& p, int kt, int tid, Staged<BM, NT>& r) {
  constexpr int RP = NT / 8;  // rows per pass
  constexpr int BK = Elt<T>::BK, VE = Elt<T>::VE;
  constexpr bool IS_16BIT = sizeof(T) == 2;
  const size_t k0 = (size_t)kt * BK;
  const T* Ap = A + (size_t)(tid >> 3) * p.a_rs + k0 + (tid & 7) * VE;  // row tid/8 (+RP per pass), chunk tid%8
  const size_t a_step = (size_t)RP * p.a_rs;
#pragma unroll
  for (int i = 0; i < BM / RP; ++i) {
    if (RAGGED) {
      const int row = min((tid >> 3) + i * RP, p.M - 1);
      r.a[i] = *reinterpret_cast<const u32x4*>(A + (size_t)row * p.a_rs + k0 + (tid & 7) * VE);
    } else {
      r.a[i] = *reinterpret_cast<const u32x4*>(Ap + i * a_step);
    }
  }
  if (B_NK) {
    const size_t k0b = p.b_k_div > 1 ? (size_t)((p.b_kt0 + kt) / p.b_k_div) * BK : k0;
    const BT* Bp = B + (size_t)(tid >> 3) * p.b_cs + k0b + (tid & 7) * VE;
    const size_t b_step = (size_t)RP * p.b_cs;
#pragma unroll
    for (int i = 0; i < BN / RP; ++i) {
      if (RAGGED) {
        const int row = min((tid >> 3) + i * RP, p.n_tile - 1);
        const BT* q = B + (size_t)row * p.b_cs + k0b + (tid & 7) * VE;
        if (B_NK == 2) {
          const u32x2 v = *reinterpret_cast<const u32x2*>(q);
          r.b[i].x = v.x;
          r.b[i].y = v.y;
        } else {
          r.b[i] = *reinterpret_cast<const u32x4*>(q);
        }
      } else if (B_NK == 2) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(Bp + i * b_step);
        r.b[i].x = v.x;
        r.b[i].y = v.y;
      } else {
        r.b[i] = *reinterpret_cast<const u32x4*>(Bp + i * b_step);
      }
    }
  } else if (tid < 2 * BN) {
    // 4 (k) x 8 (n) bf16 block or 4 (k) x 4 (n) f32 block per thread; 2 * BN threads cover the tile
    const int kg = IS_16BIT ? (tid & 15) : (tid & 7), ng = IS_16BIT ? (tid >> 4) : (tid >> 3);
    const T* Bp = reinterpret_cast<const T*>(B) + (k0 + kg * 4) * (size_t)p.b_rs + ng * VE;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.b[i] = *reinterpret_cast<const u32x4*>(Bp + i * (size_t)p.b_rs);
  }
}

// Staging stores of one prefetched tile, split into four parts (PART = 0..3) so that they can be
// spread between the MFMAs of a K tile.  PART < 0 issues all of them.
template <typename T, int B_NK, int BM, int BN, int NT, int PART>
__device__ __forceinline__ void store_tiles(u32x4* __restrict__ S, int tid, const Staged<BM, NT>& r) {
  constexpr bool IS_16BIT = sizeof(T) == 2;
  constexpr int RP = NT / 8, NA = BM / RP;
  const int row = tid >> 3, chunk = tid & 7;  // rows RP (32 or 64) apart share one swizzle
  u32x4* Sa = S + row * CHUNKS + (chunk ^ lds_swz(row));
#pragma unroll
  for (int i = 0; i < NA; ++i)
    if (PART < 0 || (i & 3) == PART) Sa[i * RP * CHUNKS] = r.a[i];
  if (B_NK) {
    u32x4* Sb = Sa + BM * CHUNKS;
#pragma unroll
    for (int i = 0; i < BN / RP; ++i)
      if (PART < 0 || ((NA + i) & 3) == PART) Sb[i * RP * CHUNKS] = B_NK == 2 ? widen_bf16x4(r.b[i]) : r.b[i];
  } else if (tid < 2 * BN) {
    if (IS_16BIT) {
      const int kg = tid & 15, ng = tid >> 4;
      u32x2* S2 = reinterpret_cast<u32x2*>(S);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (PART < 0 || (j & 3) == PART) {
          // column j of the 4 x 8 block: rows (k, k+1) and (k+2, k+3) packed as two dwords
          const unsigned sel = (j & 1) ? 0x07060302u : 0x05040100u;
          u32x2 v;
          v.x = __builtin_amdgcn_perm(r.b[1][j >> 1], r.b[0][j >> 1], sel);
          v.y = __builtin_amdgcn_perm(r.b[3][j >> 1], r.b[2][j >> 1], sel);
          S2[lds_idx(BM + ng * 8 + j, kg >> 1) * 2 + (kg & 1)] = v;
        }
      }
    } else {
      const int kg = tid & 7, ng = tid >> 3;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (PART < 0 || j == PART) S[lds_idx(BM + ng * 4 + j, kg)] = u32x4{r.b[0][j], r.b[1][j], r.b[2][j], r.b[3][j]};
    }
  }
}

// MFMA operands of one 16-wide (bf16) / 8-wide (f32) k step of the wave's tile.
template <int MI, int NJ>
struct Frags {
  u32x4 a[MI], b[NJ];
};

template <int BM, int MI, int NJ>
__device__ __forceinline__ void load_frags(const u32x4* __restrict__ S, int lane, int wm, int wn, int s, Frags<MI, NJ>& f) {
  const int chunk = 2 * s + (lane >> 5);
#pragma unroll
  for (int i = 0; i < MI; ++i) f.a[i] = S[lds_idx(wm + i * 32 + (lane & 31), chunk)];
#pragma unroll
  for (int j = 0; j < NJ; ++j) f.b[j] = S[lds_idx(BM + wn + j * 32 + (lane & 31), chunk)];
}

template <typename T, int MI, int NJ>
__device__ __forceinline__ void mma_frags(const Frags<MI, NJ>& f, floatx16 (&acc)[MI][NJ]) {
  constexpr bool IS_16BIT = sizeof(T) == 2;
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (IS_16BIT) {
        acc[i][j] = mma16(T(), f.a[i], f.b[j], acc[i][j]);
      } else {
        // whole-vector casts: __builtin_bit_cast applied to one element of an ext vector reads element 0
        const f32x4 af = __builtin_bit_cast(f32x4, f.a[i]), bf = __builtin_bit_cast(f32x4, f.b[j]);
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.x, bf.x, acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.y, bf.y, acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.z, bf.z, acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.w, bf.w, acc[i][j], 0, 0, 0);
      }
    }
}

// Issue order of one k step, as scheduling groups: every MFMA is followed by its share of the step's
// memory instructions (LDS reads of the next step first, then staging stores, global loads spread
// in between), so that each of them issues in the shadow of a running MFMA instead of in a burst
// that fills the LDS queue and blocks the wave.
template <int N_MFMA, int N_READ, int N_WRITE, int N_VMEM>
__device__ __forceinline__ void interleave_step() {
  constexpr int N_DS = N_READ + N_WRITE;
#pragma unroll
  for (int i = 0; i < N_MFMA; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
#pragma unroll
    for (int d = i * N_DS / N_MFMA; d < (i + 1) * N_DS / N_MFMA; ++d) {
      if (d < N_READ) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      else __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);             // one LDS write
    }
#pragma unroll
    for (int v = i * N_VMEM / N_MFMA; v < (i + 1) * N_VMEM / N_MFMA; ++v) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
  }
}

// Staging stores of part PART (see store_tiles): A stores i with i % 4 == PART, then B's.
template <typename T, int B_NK, int BM, int BN, int NT>
constexpr int stores_in_part(int part) {
  const int rp = NT / 8, na = BM / rp;
  int n = 0;
  for (int i = 0; i < na; ++i) n += (i & 3) == part;
  if (B_NK) {
    for (int i = 0; i < BN / rp; ++i) n += ((na + i) & 3) == part;
  } else if (sizeof(T) == 2) {
    n += 2;  // 8 columns, two per part
  } else {
    n += 1;  // 4 columns, one per part
  }
  return n;
}

// One K tile: multiply the tile in LDS stage `cur`; meanwhile move the tile held in `wr` (loaded
// from global memory one phase ago) into stage `nxt`, a quarter per k step, and start the global
// loads of tile `load_kt` into `ld`.  Fragments are double-buffered in registers: the LDS reads of
// k step s+1 are in flight while the MFMAs of step s run.
// WRITE: 1 = always store, 0 = never, 2 = decided at run time by `do_write` (tail phases; a
// run-time branch splits the scheduling region, so the steady state uses the compile-time forms).
// The loads are unconditional (LOAD is a compile-time switch): a load under a run-time branch makes
// the compiler wait for every outstanding load before the staging stores, which would undo the
// two-tile lead.
template <typename T, int B_NK, int BM, int BN, int NT, int MI, int NJ, bool LOAD, int WRITE, bool RAGGED = false>
__device__ __forceinline__ void k_phase(const T* __restrict__ A, const typename RhsElt<T, B_NK>::type* __restrict__ B, const MMArgs& p, const u32x4* __restrict__ cur, u32x4* __restrict__ nxt,
                                        bool do_write, const Staged<BM, NT>& wr, int load_kt, Staged<BM, NT>& ld, int tid, int lane, int wm, int wn,
                                        floatx16 (&acc)[MI][NJ]) {
  constexpr int N_MFMA = MI * NJ * (sizeof(T) == 4 ? 4 : 1), N_READ = MI + NJ;
  constexpr int N_VMEM = LOAD ? BM * 8 / NT + (B_NK ? BN * 8 / NT : 4) : 0;
  constexpr bool FINE = WRITE != 2;
  Frags<MI, NJ> f0, f1;
  load_frags<BM, MI, NJ>(cur, lane, wm, wn, 0, f0);
  __builtin_amdgcn_sched_barrier(0);
  // step 0
  if (LOAD) load_tiles<T, B_NK, BM, BN, NT, RAGGED>(A, B, p, load_kt, tid, ld);
  load_frags<BM, MI, NJ>(cur, lane, wm, wn, 1, f1);
  mma_frags<T, MI, NJ>(f0, acc);
  if (WRITE == 1 || (WRITE == 2 && do_write)) store_tiles<T, B_NK, BM, BN, NT, 0>(nxt, tid, wr);
  if (FINE) interleave_step<N_MFMA, N_READ, WRITE ? stores_in_part<T, B_NK, BM, BN, NT>(0) : 0, N_VMEM>();
  __builtin_amdgcn_sched_barrier(0);
  // step 1
  load_frags<BM, MI, NJ>(cur, lane, wm, wn, 2, f0);
  mma_frags<T, MI, NJ>(f1, acc);
  if (WRITE == 1 || (WRITE == 2 && do_write)) store_tiles<T, B_NK, BM, BN, NT, 1>(nxt, tid, wr);
  if (FINE) interleave_step<N_MFMA, N_READ, WRITE ? stores_in_part<T, B_NK, BM, BN, NT>(1) : 0, 0>();
  __builtin_amdgcn_sched_barrier(0);
  // step 2
  load_frags<BM, MI, NJ>(cur, lane, wm, wn, 3, f1);
  mma_frags<T, MI, NJ>(f0, acc);
  if (WRITE == 1 || (WRITE == 2 && do_write)) store_tiles<T, B_NK, BM, BN, NT, 2>(nxt, tid, wr);
  if (FINE) interleave_step<N_MFMA, N_READ, WRITE ? stores_in_part<T, B_NK, BM, BN, NT>(2) : 0, 0>();
  __builtin_amdgcn_sched_barrier(0);
  // step 3
  mma_frags<T, MI, NJ>(f1, acc);
  if (WRITE == 1 || (WRITE == 2 && do_write)) store_tiles<T, B_NK, BM, BN, NT, 3>(nxt, tid, wr);
  if (FINE) interleave_step<N_MFMA, 0, WRITE ? stores_in_part<T, B_NK, BM, BN, NT>(3) : 0, 0>();
}

// NT threads = NT / 64 waves laid out (NT / 128) x 2 over the tile: 4 waves give each wave a
// (BM/2) x (BN/2) block; 8 waves halve the rows per wave and put two waves on every SIMD, so that
// one can feed the matrix pipe while the other is blocked on the LDS or load queues.
//
// SPLIT: the K tiles are dealt to `nsplit` workgroups per output tile (slab s takes tiles
// [s * kt_per, (s + 1) * kt_per)), each writes its f32 partial tile to ws[s][batch][m][n], and
// gemm_split_reduce adds the slabs in index order.  For skinny products (few output tiles, long K:
// the projections of a 128-token prefill) this is what puts every CU to work.
template <typename T, int B_NK, int BM, int BN, int NT, bool SPLIT, bool RAGGED = false>
__global__ void __launch_bounds__(NT) gemm_tiled(MMArgs p_in, int tiles_m, int tiles_n, int remap, int nsplit, int kt_per, float* __restrict__ ws) {
  extern __shared__ u32x4 lds[];
  constexpr int BK = Elt<T>::BK;
  // waves over the tile: two columns of waves, except for a 32-row tile, whose waves sit side by side
  constexpr int WAVES_M = BM >= 64 ? NT / 128 : 1, WAVES_N = NT / 64 / WAVES_M;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, MI = WM / 32, NJ = WN / 32;
  constexpr int STAGE = (BM + BN) * CHUNKS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int bid = blockIdx.x;
  if (remap) bid = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
  int slab = 0;
  if (SPLIT) {
    slab = bid % nsplit;  // the slabs of one tile sit next to each other: they share the A and B rows
    bid /= nsplit;
  }
  const int tpb = tiles_m * tiles_n;
  const int batch = bid / tpb;
  const int t_in = bid - batch * tpb;
  const int m0 = (t_in / tiles_n) * BM, n0 = (t_in % tiles_n) * BN;
  // p: the problem as this tile sees it -- with RAGGED, M counts the rows of this tile that exist
  MMArgs p = p_in;
  if (RAGGED) {
    p.M = min(BM, p_in.M - m0);
    p.n_tile = min(BN, p_in.N - n0);
  }
  const int kt0 = SPLIT ? slab * kt_per : 0;
  const size_t k_off = (size_t)kt0 * BK;
  const T* __restrict__ A = static_cast<const T*>(p.a) + (size_t)batch * p.a_bs + (size_t)m0 * p.a_rs + k_off;
  typedef typename RhsElt<T, B_NK>::type BT;
  const size_t k_off_b = B_NK && p.b_k_div > 1 ? 0 : k_off;  // an rhs that meets several lhs tiles per tile is addressed from its first K tile
  p.b_kt0 = kt0;
  const BT* __restrict__ B =
      static_cast<const BT*>(p.b) + (size_t)batch * p.b_bs + (B_NK ? (size_t)n0 * p.b_cs + k_off_b : (size_t)n0 + k_off_b * (size_t)p.b_rs);
  const int KT = SPLIT ? min(kt_per, p.K / BK - kt0) : p.K / BK;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;

  floatx16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Global loads run two tiles ahead of the MFMAs: tile kt+2 is on its way into one register set
  // while tile kt+1 moves from the other set into the idle LDS stage and tile kt is multiplied.
  Staged<BM, NT> r0, r1;
  u32x4* lds0 = lds;
  u32x4* lds1 = lds + STAGE;
  load_tiles<T, B_NK, BM, BN, NT, RAGGED>(A, B, p, 0, tid, r0);
  if (KT > 1) load_tiles<T, B_NK, BM, BN, NT, RAGGED>(A, B, p, 1, tid, r1);
  store_tiles<T, B_NK, BM, BN, NT, -1>(lds0, tid, r0);
  __syncthreads();
  int kt = 0;
  // steady state: both phases store and load unconditionally (tiles kt+2 and kt+3 exist)
  for (; kt + 3 < KT; kt += 2) {
    // stage 1 was last read in the previous odd phase, a barrier ago
    k_phase<T, B_NK, BM, BN, NT, MI, NJ, true, 1, RAGGED>(A, B, p, lds0, lds1, true, r1, kt + 2, r0, tid, lane, wm, wn, acc);
    __syncthreads();
    k_phase<T, B_NK, BM, BN, NT, MI, NJ, true, 1, RAGGED>(A, B, p, lds1, lds0, true, r0, kt + 3, r1, tid, lane, wm, wn, acc);
    __syncthreads();
  }
  // the last two or three tiles: tile kt+2, if there is one, still has to be fetched (past the end
  // the last tile is loaded again and never stored)
  for (; kt + 1 < KT; kt += 2) {
    k_phase<T, B_NK, BM, BN, NT, MI, NJ, true, 1, RAGGED>(A, B, p, lds0, lds1, true, r1, min(kt + 2, KT - 1), r0, tid, lane, wm, wn, acc);
    __syncthreads();
    k_phase<T, B_NK, BM, BN, NT, MI, NJ, false, 2, RAGGED>(A, B, p, lds1, lds0, kt + 2 < KT, r0, 0, r1, tid, lane, wm, wn, acc);
    __syncthreads();
  }
  if (kt < KT) k_phase<T, B_NK, BM, BN, NT, MI, NJ, false, 0, RAGGED>(A, B, p, lds0, lds1, false, r1, 0, r0, tid, lane, wm, wn, acc);  // odd tile count: the last tile

  // accumulator register r of lane l: row (r/4)*8 + (l/32)*4 + r%4, column l%32
  if (SPLIT) {
    float* __restrict__ W = ws + ((size_t)slab * (gridDim.x / (nsplit * tpb)) + batch) * (size_t)p_in.M * p.N + (size_t)m0 * p.N + n0;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        float* Wt = W + (size_t)(wm + i * 32 + (lane >> 5) * 4) * p.N + wn + j * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (!RAGGED || (wm + i * 32 + (lane >> 5) * 4 + (r >> 2) * 8 + (r & 3) < p.M && wn + j * 32 + (lane & 31) < p.n_tile))
            Wt[(size_t)((r >> 2) * 8 + (r & 3)) * p.N] = acc[i][j][r];
      }
  } else {
    T* __restrict__ C = static_cast<T*>(p.c) + (size_t)batch * p.c_bs + (size_t)m0 * p.N + n0;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        T* Ct = C + (size_t)(wm + i * 32 + (lane >> 5) * 4) * p.N + wn + j * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (!RAGGED || (wm + i * 32 + (lane >> 5) * 4 + (r >> 2) * 8 + (r & 3) < p.M && wn + j * 32 + (lane & 31) < p.n_tile))
            Ct[(size_t)((r >> 2) * 8 + (r & 3)) * p.N] = (T)acc[i][j][r];
      }
  }
}

// c[i] = (T)(ws[0][i] + ws[1][i] + ... in slab order); n4 groups of 4 elements.
// EPI = GemmEpilogue::ADD: + residual[i].  EPI = GemmEpilogue::SWIGLU: the rows of the product are n wide and c's rows n / 2:
// c[r][j] = silu(sum[r][j]) * sum[r][n / 2 + j]; n4 then counts groups of 4 elements of c (x / (1 + exp(-x)), the form the lazy graph
// of ug-llama/src/model.rs:44-52 computes).
template <typename T, int EPI>
__global__ void __launch_bounds__(256) gemm_split_reduce(const float* __restrict__ ws, T* __restrict__ c, size_t n4, size_t slab_elems, int nsplit,
                                                         const float* __restrict__ residual, int n) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  f32x4 s;
  if constexpr (EPI == GemmEpilogue::SWIGLU) {
    const size_t half4 = (size_t)n / 8, r = g / half4, j4 = g % half4;  // groups of 4 per row of c
    const size_t gate = r * ((size_t)n / 4) + j4, up = gate + half4;
    f32x4 a = reinterpret_cast<const f32x4*>(ws)[gate], b = reinterpret_cast<const f32x4*>(ws)[up];
    for (int k = 1; k < nsplit; ++k) {
      a += reinterpret_cast<const f32x4*>(ws + (size_t)k * slab_elems)[gate];
      b += reinterpret_cast<const f32x4*>(ws + (size_t)k * slab_elems)[up];
    }
    s.x = a.x / (1.f + expf(-a.x)) * b.x;
    s.y = a.y / (1.f + expf(-a.y)) * b.y;
    s.z = a.z / (1.f + expf(-a.z)) * b.z;
    s.w = a.w / (1.f + expf(-a.w)) * b.w;
  } else {
    s = reinterpret_cast<const f32x4*>(ws)[g];
    for (int k = 1; k < nsplit; ++k) s += reinterpret_cast<const f32x4*>(ws + (size_t)k * slab_elems)[g];
    if constexpr (EPI == GemmEpilogue::ADD) s += reinterpret_cast<const f32x4*>(residual)[g];
  }
  T* o = c + g * 4;
  o[0] = (T)s.x;
  o[1] = (T)s.y;
  o[2] = (T)s.z;
  o[3] = (T)s.w;
}

// Raises the kernel's dynamic LDS limit once per device (`done`: one bit per device ordinal; devices past 63 pay the call every launch).
hipError_t allow_lds(const void* kernel, int lds_bytes, std::atomic<unsigned long long>& done) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
  if (bit && (done.load(std::memory_order_relaxed) & bit)) return hipSuccess;
  if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes)) return e;
  done.fetch_or(bit, std::memory_order_relaxed);
  return hipSuccess;
}

template <typename T, int B_NK, int BM, int BN, int NT, bool SPLIT, bool RAGGED = false>
hipError_t launch(hipStream_t stream, const MMArgs& p, size_t batch, int nsplit, float* ws, const GemmEpilogue* epi) {
  constexpr int LDS_BYTES = 2 * (BM + BN) * CHUNKS * 16;
  constexpr int BK = Elt<T>::BK;
  static std::atomic<unsigned long long> configured{0};  // one bit per device: the attribute is per device
  auto kernel = gemm_tiled<T, B_NK, BM, BN, NT, SPLIT, RAGGED>;
  if (hipError_t e = allow_lds(reinterpret_cast<const void*>(kernel), LDS_BYTES, configured)) return e;
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int kt = p.K / BK, kt_per = SPLIT ? (kt + nsplit - 1) / nsplit : kt;
  if (SPLIT) nsplit = (kt + kt_per - 1) / kt_per;  // no empty slab
  const size_t total = batch * (size_t)tiles_m * tiles_n * (SPLIT ? nsplit : 1);
  const int remap = !SPLIT && total % 8 == 0 ? 1 : 0;
  kernel<<<dim3((unsigned)total), dim3(NT), LDS_BYTES, stream>>>(p, tiles_m, tiles_n, remap, nsplit, kt_per, ws);
  if (hipError_t e = hipGetLastError()) return e;
  if (SPLIT) {
    const size_t elems = batch * (size_t)p.M * p.N;  // contiguous [batch, M, N] result: c_bs == M * N
    const dim3 grid((unsigned)((elems / 4 + 255) / 256)), half_grid((unsigned)((elems / 8 + 255) / 256));
    if (std::is_same<T, float>::value || (epi && epi->out_f32)) {
      float* c = static_cast<float*>(p.c);
      if (epi && epi->kind == GemmEpilogue::ADD)
        gemm_split_reduce<float, GemmEpilogue::ADD><<<grid, dim3(256), 0, stream>>>(ws, c, elems / 4, elems, nsplit, epi->residual, p.N);
      else if (epi && epi->kind == GemmEpilogue::SWIGLU)
        gemm_split_reduce<float, GemmEpilogue::SWIGLU><<<half_grid, dim3(256), 0, stream>>>(ws, c, elems / 8, elems, nsplit, nullptr, p.N);
      else
        gemm_split_reduce<float, 0><<<grid, dim3(256), 0, stream>>>(ws, c, elems / 4, elems, nsplit, nullptr, p.N);
    } else {
      if (epi) return hipErrorInvalidValue;
      gemm_split_reduce<T, 0><<<grid, dim3(256), 0, stream>>>(ws, static_cast<T*>(p.c), elems / 4, elems, nsplit, nullptr, p.N);
    }
    return hipGetLastError();
  }
  return hipSuccess;
}

template <typename T, int B_NK, bool SPLIT>
hipError_t launch_shape(hipStream_t stream, const MMArgs& p, size_t batch, int shape, int nsplit, float* ws, const GemmEpilogue* epi = nullptr) {
  switch (shape) {
    case 0:
      return tune_on(TUNE_GEMM_4WAVES) ? launch<T, B_NK, 256, 128, 256, SPLIT>(stream, p, batch, nsplit, ws, epi)
                                         : launch<T, B_NK, 256, 128, 512, SPLIT>(stream, p, batch, nsplit, ws, epi);
    case 1:
      return p.M % 128 || p.N % 128 ? launch<T, B_NK, 128, 128, 256, SPLIT, true>(stream, p, batch, nsplit, ws, epi)
                                    : launch<T, B_NK, 128, 128, 256, SPLIT>(stream, p, batch, nsplit, ws, epi);
    case 2:
      return p.M % 128 || p.N % 64 ? launch<T, B_NK, 128, 64, 256, SPLIT, true>(stream, p, batch, nsplit, ws, epi)
                                   : launch<T, B_NK, 128, 64, 256, SPLIT>(stream, p, batch, nsplit, ws, epi);
    case 3:
      return p.M % 64 || p.N % 128 ? launch<T, B_NK, 64, 128, 256, SPLIT, true>(stream, p, batch, nsplit, ws, epi)
                                   : launch<T, B_NK, 64, 128, 256, SPLIT>(stream, p, batch, nsplit, ws, epi);
    default:
      return p.M % 32 || p.N % 128 ? launch<T, B_NK, 32, 128, 256, SPLIT, true>(stream, p, batch, nsplit, ws, epi)
                                   : launch<T, B_NK, 32, 128, 256, SPLIT>(stream, p, batch, nsplit, ws, epi);
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

constexpr int kNumShapes = 5;
constexpr int kShapes[kNumShapes][2] = {{256, 128}, {128, 128}, {128, 64}, {64, 128}, {32, 128}};

// Which of the tiles a problem can take: the 128- and 64-row tiles also take an lhs whose last tile is partly empty (any
// M >= 9: fewer rows are the GEMV kernels' job) and, with an [n, k]-major rhs, an N they do not divide.  The 64-row tile
// and the 32-row tile are for prompts of up to 64 and 32 positions: most rows of a 128-row tile would be multiplied for
// nothing.
bool shape_fits(const MMArgs& p, int s) {
  // at most two tile rows: stacked higher they read every weight once per tile row and feed the pipe worse per flop
  // (1900 rows of gate|up on 32-row tiles: 778 us against 756 on 128-row ones, where the tile count alone said 692)
  if (s >= 3 && p.M > 2 * kShapes[s][0]) return false;
  const bool rhs_nk = p.b_rs == 1 && p.b_cs != 1, ragged_ok = kShapes[s][0] <= 128;
  return !((p.M % kShapes[s][0] && !ragged_ok) || (p.N % kShapes[s][1] && !(ragged_ok && rhs_nk)));
}
size_t tile_count(const MMArgs& p, size_t batch, int s) {
  return batch * (size_t)((p.M + kShapes[s][0] - 1) / kShapes[s][0]) * (size_t)((p.N + kShapes[s][1] - 1) / kShapes[s][1]);
}

// How many K slabs per output tile, and what the launch then costs (us).  A launch takes as long as its busiest CU:
// with ns slabs per tile the tiles * ns workgroups go round the 256 CUs ceil(tiles * ns / 256) times, each multiplying
// ceil(kt / ns) K tiles, and the fold moves every slab twice behind a launch of its own.  The times of the prefill
// products (128 rows against 2048..32000 x 2048..5632, f32 and three-term bf16) follow this to 10 %: 32 tiles take 8
// slabs (one workgroup per CU), 40 take 6, 176 take 4.
struct Split {
  int nsplit;
  double cost_us;
};
Split pick_split(int dtype, const MMArgs& p, size_t batch, int shape, bool always_fold = false) {
  const int bk = dtype == UGHIP_F32 ? 32 : 64;
  const size_t tiles = tile_count(p, batch, shape);
  const int kt = p.K / bk;
  // one K tile of a workgroup alone on its CU: f32 scales with the tile, the 16-bit 128x128 tile is better fed than two
  // 128x64 ones; a [k, n]-major rhs is transposed on its way to LDS
  const double area = (kShapes[shape][0] * kShapes[shape][1]) / 8192.0;
  const double tile_us = (dtype == UGHIP_F32 ? 1.03 * area : area <= 1.0 ? 0.4 : 0.325 * area) * (p.b_cs == 1 ? 1.35 : 1.0);
  const double slab_us = 2.0 * (double)batch * p.M * p.N * 4 / 5e6, fold_us = 5.0;
  Split best{1, (double)((tiles + 255) / 256) * kt * tile_us + (always_fold ? slab_us + fold_us : 0.0)};  // an epilogue folds even one slab
  if (long long v; tune_get(TUNE_GEMM_SPLIT, &v)) return Split{std::max(1, (int)v), best.cost_us};  // tuning aid
  // only when the tiles alone leave CUs idle and K is long enough that every slab still has a few tiles to pipeline; the
  // fold of the partial tiles works on groups of 4 elements
  if (tiles >= 256 || kt < 8 || (batch * (size_t)p.M * (size_t)p.N) % 4 != 0) return best;
  const int max_split = std::min(32, kt / 4);  // at least 4 K tiles per slab
  for (int ns = 2; ns <= max_split; ++ns) {
    const int kt_per = (kt + ns - 1) / ns;
    if ((kt + kt_per - 1) / kt_per != ns) continue;  // the launch would drop the empty slabs: same as a smaller ns
    const double cost = (double)((tiles * ns + 255) / 256) * kt_per * tile_us + ns * slab_us + fold_us;
    if (cost < best.cost_us) best = Split{ns, cost};
  }
  return best;
}

// The tile the cost model above makes cheapest among those that fit the problem.  Within 3 % of each other the smaller
// tile wins when both leave CUs idle unsplit (fewer than 256 tiles: more workgroups to spread), the larger one otherwise
// (fewer operand bytes per flop).  Counting rounds of 256 workgroups, not just "at least 256 tiles", is what sends
// 3072 x 4096 x 4096 f32 to 128 x 128 (768 tiles, three full rounds: 889 us) instead of 256 x 128 (384 tiles, a round and
// a half: 1000 us) and 2304^3 away from 324 tiles of 128 x 128 (303 -> 255 us).  -1: no tile fits M x N.
int pick_shape(const MMArgs& p, size_t batch, int dtype, bool always_fold = false) {
  // UGHIP_GEMM_SHAPE=0..2 forces a tile shape (tuning aid); ignored when it does not fit the problem.
  if (long long tv; tune_get(TUNE_GEMM_SHAPE, &tv)) {
    const int v = (int)tv, s = v == 6 ? 3 : v == 7 ? 4 : v;  // 3..5 name the other kernel's tiles: 6 and 7 are the 64- and 32-row tiles here
    if (s >= 0 && s < kNumShapes && (s < 3 || v >= 6) && shape_fits(p, s)) return s;
  }
  int best = -1;
  double best_cost = 0;
  for (int s = 0; s < kNumShapes; ++s) {
    if (!shape_fits(p, s)) continue;
    const double cost = pick_split(dtype, p, batch, s, always_fold).cost_us;
    if (best < 0) {
      best = s, best_cost = cost;
      continue;
    }
    // 64 x 128 against 128 x 64 (the same area): only when it is really cheaper, i.e. when the rows fit 64 -- two tile
    // rows of 64 read every weight twice
    const bool few = s < 3 && tile_count(p, batch, best) < 256 && tile_count(p, batch, s) < 256;
    if (few ? cost <= best_cost * 1.03 : cost < best_cost * 0.97) best = s, best_cost = cost;
  }
  return best;
}

}  // namespace

bool gemm_tiled_supported(int dtype, const MMArgs& p, size_t batch, bool rhs_bf16) {
  if (dtype != UGHIP_F32 && dtype != UGHIP_BF16 && dtype != UGHIP_F16) return false;
  if (rhs_bf16 && (dtype != UGHIP_F32 || p.b_rs != 1 || p.b_cs == 1)) return false;  // widening is built for an [n, k]-major rhs under an f32 product
  const int ve = dtype == UGHIP_F32 ? 4 : 8, bk = dtype == UGHIP_F32 ? 32 : 64;
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || p.K % bk || batch == 0) return false;
  if (p.a_cs != 1 || p.a_rs % ve || (batch > 1 && (p.a_bs % ve || p.b_bs % ve))) return false;  // 128-bit loads; the result is stored element by element
  const bool nn = p.b_cs == 1, nt = p.b_rs == 1;
  if (nn == nt) return false;
  if (nn && p.b_rs % ve) return false;
  if (nt && p.b_cs % ve) return false;
  if (!aligned16(p.a) || !aligned16(p.b) || !aligned16(p.c)) return false;
  const int s = pick_shape(p, batch, dtype);
  if (s < 0) return false;
  return batch * (size_t)((p.M + kShapes[s][0] - 1) / kShapes[s][0]) * (size_t)((p.N + kShapes[s][1] - 1) / kShapes[s][1]) < (1u << 24);
}

hipError_t gemm_fold_f32(hipStream_t stream, const float* slabs, float* c, size_t m, size_t n, int nsplit, GemmEpilogue::Kind kind, const float* residual) {
  const size_t elems = m * n;  // of one slab; with SwiGLU c has half of them
  if (elems == 0) return hipSuccess;
  const dim3 grid((unsigned)((elems / 4 + 255) / 256)), half_grid((unsigned)((elems / 8 + 255) / 256));
  if (kind == GemmEpilogue::SWIGLU) gemm_split_reduce<float, GemmEpilogue::SWIGLU><<<half_grid, dim3(256), 0, stream>>>(slabs, c, elems / 8, elems, nsplit, nullptr, (int)n);
  else if (kind == GemmEpilogue::ADD) gemm_split_reduce<float, GemmEpilogue::ADD><<<grid, dim3(256), 0, stream>>>(slabs, c, elems / 4, elems, nsplit, residual, (int)n);
  else gemm_split_reduce<float, 0><<<grid, dim3(256), 0, stream>>>(slabs, c, elems / 4, elems, nsplit, nullptr, (int)n);
  return hipGetLastError();
}

double gemm_tiled_cost_us(int dtype, const MMArgs& p, size_t batch) {
  if (!gemm_tiled_supported(dtype, p, batch)) return -1.0;
  const int s = pick_shape(p, batch, dtype);
  const size_t tiles = tile_count(p, batch, s);
  const double launch_us = 4.0;
  if (tiles < 256) return launch_us + pick_split(dtype, p, batch, s).cost_us;
  // many tiles: a last, partly filled round of workgroups costs a third of a full one plus its share of the rest
  // (16-bit products of 1900..5120 rows with 300, 320, 324, 384, 484 and 800 tiles: within 10 %)
  const double whole = pick_split(dtype, p, batch, s).cost_us / (double)((tiles + 255) / 256);
  const size_t part = tiles % 256;
  return launch_us + whole * ((double)(tiles / 256) + (part ? 0.35 + 0.65 * (double)part / 256.0 : 0.0));
}

size_t gemm_tiled_workspace_bytes(int dtype, const MMArgs& p, size_t batch, const GemmEpilogue* epi) {
  const int s = pick_shape(p, batch, dtype, epi != nullptr);
  if (s < 0) return 0;
  const int nsplit = pick_split(dtype, p, batch, s, epi != nullptr).nsplit;
  return nsplit > 1 || epi ? (size_t)nsplit * batch * (size_t)p.M * p.N * sizeof(float) : 0;
}

void gemm_tiled_name(int dtype, const MMArgs& p, size_t batch, bool rhs_bf16, const GemmEpilogue* epi, char* out, size_t out_len) {
  const bool nt = p.b_rs == 1 && p.b_cs != 1;
  const int s = pick_shape(p, batch, dtype, epi != nullptr);
  if (s < 0) {
    snprintf(out, out_len, "gemm_tiled<does not take this product>");
    return;
  }
  const int nsplit = pick_split(dtype, p, batch, s, epi != nullptr).nsplit;
  const char* tn = rhs_bf16 ? "f32xbf16" : dtype == UGHIP_F32 ? "f32" : dtype == UGHIP_F16 ? "f16" : "bf16";
  const bool ragged = s != 0 && (p.M % kShapes[s][0] || p.N % kShapes[s][1]);
  char split[48] = "";
  if (nsplit > 1 || epi)
    snprintf(split, sizeof split, ",splitK=%d%s%s", nsplit, !epi ? "" : epi->kind == GemmEpilogue::ADD ? ",+residual" : epi->kind == GemmEpilogue::SWIGLU ? ",swiglu" : "",
             epi && epi->out_f32 ? ",f32 out" : "");
  snprintf(out, out_len, "gemm_tiled<%s,%s,%dx%d,%dt%s%s>", tn, nt ? "NT" : "NN", kShapes[s][0], kShapes[s][1], s == 0 && !tune_on(TUNE_GEMM_4WAVES) ? 512 : 256,
           ragged ? ",ragged" : "", split);
}

hipError_t gemm_tiled_launch(hipStream_t stream, int dtype, const MMArgs& p, size_t batch, float* workspace, bool rhs_bf16, const GemmEpilogue* epi) {
  const bool nt = p.b_rs == 1 && p.b_cs != 1;
  if (rhs_bf16 && (dtype != UGHIP_F32 || !nt)) return hipErrorInvalidValue;
  // an epilogue writes f32: an f32 product, or a bf16 one ([n, k]-major rhs) whose fold is told to
  if (epi && ((dtype != UGHIP_F32 && !(dtype == UGHIP_BF16 && epi->out_f32 && nt)) || (batch * (size_t)p.M * (size_t)p.N) % 8 != 0 || p.N % 8 != 0)) return hipErrorInvalidValue;
  if (p.b_k_div > 1 && !nt) return hipErrorInvalidValue;
  const int s = pick_shape(p, batch, dtype, epi != nullptr);
  if (s < 0) return hipErrorInvalidValue;
  const int nsplit = pick_split(dtype, p, batch, s, epi != nullptr).nsplit;
  {
    char name[160];
    gemm_tiled_name(dtype, p, batch, rhs_bf16, epi, name, sizeof name);
    note_kernel("%s", name);
  }
  if (nsplit > 1 || epi) {
    if (!workspace) return hipErrorInvalidValue;
    if (rhs_bf16) return launch_shape<float, 2, true>(stream, p, batch, s, nsplit, workspace, epi);
    if (dtype == UGHIP_F32)
      return nt ? launch_shape<float, true, true>(stream, p, batch, s, nsplit, workspace, epi) : launch_shape<float, false, true>(stream, p, batch, s, nsplit, workspace, epi);
    if (dtype == UGHIP_F16)
      return nt ? launch_shape<_Float16, true, true>(stream, p, batch, s, nsplit, workspace) : launch_shape<_Float16, false, true>(stream, p, batch, s, nsplit, workspace);
    return nt ? launch_shape<__bf16, true, true>(stream, p, batch, s, nsplit, workspace, epi) : launch_shape<__bf16, false, true>(stream, p, batch, s, nsplit, workspace);
  }
  if (rhs_bf16) return launch_shape<float, 2, false>(stream, p, batch, s, 1, nullptr);
  if (dtype == UGHIP_F32)
    return nt ? launch_shape<float, true, false>(stream, p, batch, s, 1, nullptr) : launch_shape<float, false, false>(stream, p, batch, s, 1, nullptr);
  if (dtype == UGHIP_F16)
    return nt ? launch_shape<_Float16, true, false>(stream, p, batch, s, 1, nullptr) : launch_shape<_Float16, false, false>(stream, p, batch, s, 1, nullptr);
  return nt ? launch_shape<__bf16, true, false>(stream, p, batch, s, 1, nullptr) : launch_shape<__bf16, false, false>(stream, p, batch, s, 1, nullptr);
}

}  // namespace ughip
