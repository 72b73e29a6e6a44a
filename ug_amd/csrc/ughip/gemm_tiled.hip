// Tuned MFMA GEMM for gfx950: C[b] = A[b] x B[b], f32 accumulate.
//
//   block tile BM x BN (256x128, 128x128 or 128x64), 4 waves (2 x 2), each wave owns a
//   (BM/2) x (BN/2) block of MFMA 32x32 accumulators
//   K tile = 128 bytes per matrix row (64 bf16 / 32 f32), double-buffered in LDS, the next tile
//   prefetched into registers while the current one feeds the matrix cores
//   LDS rows are 8 chunks of 16 bytes, chunk' = chunk ^ (row & 7): every 128-bit fragment read and
//   every staging write is bank-conflict free
//   a row-major B ([k, n]) is transposed in registers on its way to LDS so that both MFMA
//   operands read 128 bits of consecutive k (v_perm_b32 for bf16; free for f32)
//   tiles are handed to workgroups XCD by XCD so that the tiles of one batch element share an L2
//
// bf16: v_mfma_f32_32x32x16_bf16 (lane l feeds row/col l%32, k = 8*(l/32)..+7).
// f32:  v_mfma_f32_32x32x2_f32   (lane l feeds row/col l%32, k = l/32); the 4 floats of a 128-bit
//       fragment feed 4 consecutive MFMAs, lanes 0-31 holding k..k+3 and lanes 32-63 k+4..k+7.
#include <hip/hip_runtime.h>

#include "gemm.h"
#include "ughip.h"

namespace ughip {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
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

__device__ __forceinline__ int lds_idx(int row, int chunk) { return row * CHUNKS + (chunk ^ (row & 7)); }

// The tile being prefetched from global memory while the previous one is multiplied.
template <int BM>
struct Staged {
  u32x4 a[BM / 32];
  u32x4 b[4];
};

template <typename T, bool B_NK, int BM, int BN>
__device__ __forceinline__ void load_tiles(const T* __restrict__ A, const T* __restrict__ B, const MMArgs& p, int kt, int tid, Staged<BM>& r) {
  constexpr int BK = Elt<T>::BK, VE = Elt<T>::VE;
  constexpr bool IS_BF16 = sizeof(T) == 2;
  const size_t k0 = (size_t)kt * BK;
  const T* Ap = A + (size_t)(tid >> 3) * p.a_rs + k0 + (tid & 7) * VE;  // row tid/8 (+32 per step), chunk tid%8
  const size_t a_step = (size_t)32 * p.a_rs;
#pragma unroll
  for (int i = 0; i < BM / 32; ++i) r.a[i] = *reinterpret_cast<const u32x4*>(Ap + i * a_step);
  if (B_NK) {
    const T* Bp = B + (size_t)(tid >> 3) * p.b_cs + k0 + (tid & 7) * VE;
    const size_t b_step = (size_t)32 * p.b_cs;
#pragma unroll
    for (int i = 0; i < BN / 32; ++i) r.b[i] = *reinterpret_cast<const u32x4*>(Bp + i * b_step);
  } else if (tid < 2 * BN) {
    // 4 (k) x 8 (n) bf16 block or 4 (k) x 4 (n) f32 block per thread; 2 * BN threads cover the tile
    const int kg = IS_BF16 ? (tid & 15) : (tid & 7), ng = IS_BF16 ? (tid >> 4) : (tid >> 3);
    const T* Bp = B + (k0 + kg * 4) * (size_t)p.b_rs + ng * VE;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.b[i] = *reinterpret_cast<const u32x4*>(Bp + i * (size_t)p.b_rs);
  }
}

template <typename T, bool B_NK, int BM, int BN>
__device__ __forceinline__ void store_tiles(u32x4* __restrict__ S, int tid, const Staged<BM>& r) {
  constexpr bool IS_BF16 = sizeof(T) == 2;
  const int row = tid >> 3, chunk = tid & 7;  // (row + 32 i) & 7 == row & 7: one swizzle for all steps
  u32x4* Sa = S + row * CHUNKS + (chunk ^ (row & 7));
#pragma unroll
  for (int i = 0; i < BM / 32; ++i) Sa[i * 32 * CHUNKS] = r.a[i];
  if (B_NK) {
    u32x4* Sb = Sa + BM * CHUNKS;
#pragma unroll
    for (int i = 0; i < BN / 32; ++i) Sb[i * 32 * CHUNKS] = r.b[i];
  } else if (tid < 2 * BN) {
    if (IS_BF16) {
      const int kg = tid & 15, ng = tid >> 4;
      u32x2* S2 = reinterpret_cast<u32x2*>(S);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // column j of the 4 x 8 block: rows (k, k+1) and (k+2, k+3) packed as two dwords
        const unsigned sel = (j & 1) ? 0x07060302u : 0x05040100u;
        u32x2 v;
        v.x = __builtin_amdgcn_perm(r.b[1][j >> 1], r.b[0][j >> 1], sel);
        v.y = __builtin_amdgcn_perm(r.b[3][j >> 1], r.b[2][j >> 1], sel);
        S2[lds_idx(BM + ng * 8 + j, kg >> 1) * 2 + (kg & 1)] = v;
      }
    } else {
      const int kg = tid & 7, ng = tid >> 3;
#pragma unroll
      for (int j = 0; j < 4; ++j) S[lds_idx(BM + ng * 4 + j, kg)] = u32x4{r.b[0][j], r.b[1][j], r.b[2][j], r.b[3][j]};
    }
  }
}

template <typename T, int BM, int MI, int NJ>
__device__ __forceinline__ void compute_tile(const u32x4* __restrict__ S, int lane, int wm, int wn, floatx16 (&acc)[MI][NJ]) {
  constexpr bool IS_BF16 = sizeof(T) == 2;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int chunk = 2 * s + (lane >> 5);
    u32x4 a[MI], b[NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i) a[i] = S[lds_idx(wm + i * 32 + (lane & 31), chunk)];
#pragma unroll
    for (int j = 0; j < NJ; ++j) b[j] = S[lds_idx(BM + wn + j * 32 + (lane & 31), chunk)];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (IS_BF16) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[i]), __builtin_bit_cast(bf16x8, b[j]), acc[i][j], 0, 0, 0);
        } else {
          // whole-vector casts: __builtin_bit_cast applied to one element of an ext vector reads element 0
          const f32x4 af = __builtin_bit_cast(f32x4, a[i]), bf = __builtin_bit_cast(f32x4, b[j]);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.x, bf.x, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.y, bf.y, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.z, bf.z, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af.w, bf.w, acc[i][j], 0, 0, 0);
        }
      }
  }
}

template <typename T, bool B_NK, int BM, int BN>
__global__ void __launch_bounds__(256) gemm_tiled(MMArgs p, int tiles_m, int tiles_n, int remap) {
  extern __shared__ u32x4 lds[];
  constexpr int BK = Elt<T>::BK;
  constexpr int WM = BM / 2, WN = BN / 2, MI = WM / 32, NJ = WN / 32;
  constexpr int STAGE = (BM + BN) * CHUNKS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int bid = blockIdx.x;
  if (remap) bid = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
  const int tpb = tiles_m * tiles_n;
  const int batch = bid / tpb;
  const int t_in = bid - batch * tpb;
  const int m0 = (t_in / tiles_n) * BM, n0 = (t_in % tiles_n) * BN;
  const T* __restrict__ A = static_cast<const T*>(p.a) + (size_t)batch * p.a_bs + (size_t)m0 * p.a_rs;
  const T* __restrict__ B = static_cast<const T*>(p.b) + (size_t)batch * p.b_bs + (B_NK ? (size_t)n0 * p.b_cs : (size_t)n0);
  T* __restrict__ C = static_cast<T*>(p.c) + (size_t)batch * p.c_bs + (size_t)m0 * p.N + n0;
  const int KT = p.K / BK;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

  Staged<BM> st;
  floatx16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  load_tiles<T, B_NK, BM, BN>(A, B, p, 0, tid, st);
  store_tiles<T, B_NK, BM, BN>(lds, tid, st);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = kt + 1 < KT;
    if (more) load_tiles<T, B_NK, BM, BN>(A, B, p, kt + 1, tid, st);
    compute_tile<T, BM, MI, NJ>(lds + (kt & 1) * STAGE, lane, wm, wn, acc);
    // stage (kt+1)&1 was last read during iteration kt-1; every wave has passed the barrier since
    if (more) store_tiles<T, B_NK, BM, BN>(lds + ((kt + 1) & 1) * STAGE, tid, st);
    __syncthreads();
  }

  // accumulator register r of lane l: row (r/4)*8 + (l/32)*4 + r%4, column l%32
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      T* Ct = C + (size_t)(wm + i * 32 + (lane >> 5) * 4) * p.N + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) Ct[(size_t)((r >> 2) * 8 + (r & 3)) * p.N] = (T)acc[i][j][r];
    }
}

template <typename T, bool B_NK, int BM, int BN>
hipError_t launch(hipStream_t stream, const MMArgs& p, size_t batch) {
  constexpr int LDS_BYTES = 2 * (BM + BN) * CHUNKS * 16;
  static bool configured = false;
  auto kernel = gemm_tiled<T, B_NK, BM, BN>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const int tiles_m = p.M / BM, tiles_n = p.N / BN;
  const size_t total = batch * (size_t)tiles_m * tiles_n;
  const int remap = total % 8 == 0 ? 1 : 0;
  kernel<<<dim3((unsigned)total), dim3(256), LDS_BYTES, stream>>>(p, tiles_m, tiles_n, remap);
  return hipGetLastError();
}

template <typename T, bool B_NK>
hipError_t launch_shape(hipStream_t stream, const MMArgs& p, size_t batch, int shape) {
  switch (shape) {
    case 0: return launch<T, B_NK, 256, 128>(stream, p, batch);
    case 1: return launch<T, B_NK, 128, 128>(stream, p, batch);
    default: return launch<T, B_NK, 128, 64>(stream, p, batch);
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

constexpr int kShapes[3][2] = {{256, 128}, {128, 128}, {128, 64}};

// The largest tile that divides the problem and still gives every CU a workgroup; failing that,
// the dividing tile with the most workgroups.  -1: no tile divides M x N.
int pick_shape(const MMArgs& p, size_t batch) {
  int best = -1;
  size_t best_tiles = 0;
  for (int s = 0; s < 3; ++s) {
    if (p.M % kShapes[s][0] || p.N % kShapes[s][1]) continue;
    const size_t tiles = batch * (size_t)(p.M / kShapes[s][0]) * (size_t)(p.N / kShapes[s][1]);
    if (tiles >= 256) return s;
    if (tiles > best_tiles) best = s, best_tiles = tiles;
  }
  return best;
}

}  // namespace

bool gemm_tiled_supported(int dtype, const MMArgs& p, size_t batch) {
  if (dtype != UGHIP_F32 && dtype != UGHIP_BF16) return false;
  const int ve = dtype == UGHIP_F32 ? 4 : 8, bk = dtype == UGHIP_F32 ? 32 : 64;
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || p.K % bk || batch == 0) return false;
  if (p.a_cs != 1 || p.a_rs % ve || p.a_bs % ve || p.b_bs % ve || p.c_bs % ve) return false;
  const bool nn = p.b_cs == 1, nt = p.b_rs == 1;
  if (nn == nt) return false;
  if (nn && p.b_rs % ve) return false;
  if (nt && p.b_cs % ve) return false;
  if (!aligned16(p.a) || !aligned16(p.b) || !aligned16(p.c)) return false;
  const int s = pick_shape(p, batch);
  if (s < 0) return false;
  return batch * (size_t)(p.M / kShapes[s][0]) * (size_t)(p.N / kShapes[s][1]) < (1u << 30);
}

hipError_t gemm_tiled_launch(hipStream_t stream, int dtype, const MMArgs& p, size_t batch) {
  const bool nt = p.b_rs == 1 && p.b_cs != 1;
  const int s = pick_shape(p, batch);
  if (s < 0) return hipErrorInvalidValue;
  if (dtype == UGHIP_F32) return nt ? launch_shape<float, true>(stream, p, batch, s) : launch_shape<float, false>(stream, p, batch, s);
  return nt ? launch_shape<__bf16, true>(stream, p, batch, s) : launch_shape<__bf16, false>(stream, p, batch, s);
}

}  // namespace ughip
