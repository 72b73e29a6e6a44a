// Tuned MFMA GEMM for gfx950: C[b] = A[b] x B[b], f32 accumulate.
//
//   block tile 256 x 128, 4 waves (2 x 2), each wave owns 128 x 64 = 4 x 2 MFMA 32x32 accumulators
//   K tile = 128 bytes per matrix row (64 bf16 / 32 f32), double-buffered in LDS (96 KiB), the next
//   tile prefetched into registers while the current one feeds the matrix cores
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

constexpr int BM = 256, BN = 128;
constexpr int CHUNKS = 8;  // 16-byte chunks per 128-byte LDS row
constexpr int STAGE_ROWS = BM + BN;
constexpr int LDS_BYTES = 2 * STAGE_ROWS * CHUNKS * 16;

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
struct Staged {
  u32x4 a0, a1, a2, a3, a4, a5, a6, a7, b0, b1, b2, b3;
};

template <typename T, bool B_NK>
__device__ __forceinline__ void load_tiles(const T* __restrict__ A, const T* __restrict__ B, const MMArgs& p, int kt, int tid, Staged& r) {
  constexpr int BK = Elt<T>::BK, VE = Elt<T>::VE;
  constexpr bool IS_BF16 = sizeof(T) == 2;
  const size_t k0 = (size_t)kt * BK;
  const T* Ap = A + (size_t)(tid >> 3) * p.a_rs + k0 + (tid & 7) * VE;  // row tid/8 (+32 per step), chunk tid%8
  const size_t a_step = (size_t)32 * p.a_rs;
  r.a0 = *reinterpret_cast<const u32x4*>(Ap);
  r.a1 = *reinterpret_cast<const u32x4*>(Ap + a_step);
  r.a2 = *reinterpret_cast<const u32x4*>(Ap + 2 * a_step);
  r.a3 = *reinterpret_cast<const u32x4*>(Ap + 3 * a_step);
  r.a4 = *reinterpret_cast<const u32x4*>(Ap + 4 * a_step);
  r.a5 = *reinterpret_cast<const u32x4*>(Ap + 5 * a_step);
  r.a6 = *reinterpret_cast<const u32x4*>(Ap + 6 * a_step);
  r.a7 = *reinterpret_cast<const u32x4*>(Ap + 7 * a_step);
  if (B_NK) {
    const T* Bp = B + (size_t)(tid >> 3) * p.b_cs + k0 + (tid & 7) * VE;
    const size_t b_step = (size_t)32 * p.b_cs;
    r.b0 = *reinterpret_cast<const u32x4*>(Bp);
    r.b1 = *reinterpret_cast<const u32x4*>(Bp + b_step);
    r.b2 = *reinterpret_cast<const u32x4*>(Bp + 2 * b_step);
    r.b3 = *reinterpret_cast<const u32x4*>(Bp + 3 * b_step);
  } else {
    // 4 (k) x 8 (n) bf16 block or 4 (k) x 4 (n) f32 block per thread
    const int kg = IS_BF16 ? (tid & 15) : (tid & 7), ng = IS_BF16 ? (tid >> 4) : (tid >> 3);
    const T* Bp = B + (k0 + kg * 4) * (size_t)p.b_rs + ng * VE;
    r.b0 = *reinterpret_cast<const u32x4*>(Bp);
    r.b1 = *reinterpret_cast<const u32x4*>(Bp + (size_t)p.b_rs);
    r.b2 = *reinterpret_cast<const u32x4*>(Bp + 2 * (size_t)p.b_rs);
    r.b3 = *reinterpret_cast<const u32x4*>(Bp + 3 * (size_t)p.b_rs);
  }
}

template <typename T, bool B_NK>
__device__ __forceinline__ void store_tiles(u32x4* __restrict__ S, int tid, const Staged& r) {
  constexpr bool IS_BF16 = sizeof(T) == 2;
  const int row = tid >> 3, chunk = tid & 7;  // (row + 32 i) & 7 == row & 7: one swizzle for all 8
  u32x4* Sa = S + row * CHUNKS + (chunk ^ (row & 7));
  Sa[0 * 32 * CHUNKS] = r.a0;
  Sa[1 * 32 * CHUNKS] = r.a1;
  Sa[2 * 32 * CHUNKS] = r.a2;
  Sa[3 * 32 * CHUNKS] = r.a3;
  Sa[4 * 32 * CHUNKS] = r.a4;
  Sa[5 * 32 * CHUNKS] = r.a5;
  Sa[6 * 32 * CHUNKS] = r.a6;
  Sa[7 * 32 * CHUNKS] = r.a7;
  if (B_NK) {
    u32x4* Sb = Sa + BM * CHUNKS;
    Sb[0 * 32 * CHUNKS] = r.b0;
    Sb[1 * 32 * CHUNKS] = r.b1;
    Sb[2 * 32 * CHUNKS] = r.b2;
    Sb[3 * 32 * CHUNKS] = r.b3;
  } else if (IS_BF16) {
    const int kg = tid & 15, ng = tid >> 4;
    u32x2* S2 = reinterpret_cast<u32x2*>(S);
    // column j of the 4 x 8 block: rows (k, k+1) and (k+2, k+3) packed as two dwords
#define UG_COL(j, w)                                                                              \
  {                                                                                               \
    const unsigned sel = ((j) & 1) ? 0x07060302u : 0x05040100u;                                  \
    u32x2 v;                                                                                      \
    v.x = __builtin_amdgcn_perm(r.b1.w, r.b0.w, sel);                                             \
    v.y = __builtin_amdgcn_perm(r.b3.w, r.b2.w, sel);                                             \
    S2[lds_idx(BM + ng * 8 + (j), kg >> 1) * 2 + (kg & 1)] = v;                                   \
  }
    UG_COL(0, x) UG_COL(1, x) UG_COL(2, y) UG_COL(3, y) UG_COL(4, z) UG_COL(5, z) UG_COL(6, w) UG_COL(7, w)
#undef UG_COL
  } else {
    const int kg = tid & 7, ng = tid >> 3;
    S[lds_idx(BM + ng * 4 + 0, kg)] = u32x4{r.b0.x, r.b1.x, r.b2.x, r.b3.x};
    S[lds_idx(BM + ng * 4 + 1, kg)] = u32x4{r.b0.y, r.b1.y, r.b2.y, r.b3.y};
    S[lds_idx(BM + ng * 4 + 2, kg)] = u32x4{r.b0.z, r.b1.z, r.b2.z, r.b3.z};
    S[lds_idx(BM + ng * 4 + 3, kg)] = u32x4{r.b0.w, r.b1.w, r.b2.w, r.b3.w};
  }
}

template <typename T>
__device__ __forceinline__ void compute_tile(const u32x4* __restrict__ S, int lane, int wm, int wn, floatx16 (&acc)[4][2]) {
  constexpr bool IS_BF16 = sizeof(T) == 2;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int chunk = 2 * s + (lane >> 5);
    u32x4 a[4], b[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = S[lds_idx(wm + i * 32 + (lane & 31), chunk)];
#pragma unroll
    for (int j = 0; j < 2; ++j) b[j] = S[lds_idx(BM + wn + j * 32 + (lane & 31), chunk)];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
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

template <typename T, bool B_NK>
__global__ void __launch_bounds__(256) gemm_tiled(MMArgs p, int tiles_m, int tiles_n, int remap) {
  extern __shared__ u32x4 lds[];
  constexpr int BK = Elt<T>::BK;
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
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 64;

  Staged st;
  floatx16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  load_tiles<T, B_NK>(A, B, p, 0, tid, st);
  store_tiles<T, B_NK>(lds, tid, st);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = kt + 1 < KT;
    if (more) load_tiles<T, B_NK>(A, B, p, kt + 1, tid, st);
    compute_tile<T>(lds + (kt & 1) * STAGE_ROWS * CHUNKS, lane, wm, wn, acc);
    // stage (kt+1)&1 was last read during iteration kt-1; every wave has passed the barrier since
    if (more) store_tiles<T, B_NK>(lds + ((kt + 1) & 1) * STAGE_ROWS * CHUNKS, tid, st);
    __syncthreads();
  }

  // accumulator register r of lane l: row (r/4)*8 + (l/32)*4 + r%4, column l%32
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      T* Ct = C + (size_t)(wm + i * 32 + (lane >> 5) * 4) * p.N + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) Ct[(size_t)((r >> 2) * 8 + (r & 3)) * p.N] = (T)acc[i][j][r];
    }
}

template <typename T, bool B_NK>
hipError_t launch(hipStream_t stream, const MMArgs& p, size_t batch) {
  static bool configured = false;
  auto kernel = gemm_tiled<T, B_NK>;
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

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

bool gemm_tiled_supported(int dtype, const MMArgs& p, size_t batch) {
  if (dtype != UGHIP_F32 && dtype != UGHIP_BF16) return false;
  const int ve = dtype == UGHIP_F32 ? 4 : 8, bk = dtype == UGHIP_F32 ? 32 : 64;
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || p.M % BM || p.N % BN || p.K % bk) return false;
  if (p.a_cs != 1 || p.a_rs % ve || p.a_bs % ve || p.b_bs % ve || p.c_bs % ve) return false;
  const bool nn = p.b_cs == 1, nt = p.b_rs == 1;
  if (nn == nt) return false;
  if (nn && p.b_rs % ve) return false;
  if (nt && p.b_cs % ve) return false;
  if (!aligned16(p.a) || !aligned16(p.b) || !aligned16(p.c)) return false;
  const size_t total = batch * (size_t)(p.M / BM) * (size_t)(p.N / BN);
  return total > 0 && total < (1u << 30);
}

hipError_t gemm_tiled_launch(hipStream_t stream, int dtype, const MMArgs& p, size_t batch) {
  const bool nt = p.b_rs == 1 && p.b_cs != 1;
  if (dtype == UGHIP_F32) return nt ? launch<float, true>(stream, p, batch) : launch<float, false>(stream, p, batch);
  return nt ? launch<__bf16, true>(stream, p, batch) : launch<__bf16, false>(stream, p, batch);
}

}  // namespace ughip
