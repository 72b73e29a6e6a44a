// Device::matmul for gfx950: MFMA kernels with f32 accumulation (f32 via v_mfma_f32_32x32x2_f32,
// bf16 via v_mfma_f32_32x32x16_bf16), plus a bandwidth-bound GEMV for the m <= 8 rows of decode.
// dst[b,m,n] = lhs[b,m,k] x rhs[b,k,n], beta = 0 (ug-core/src/lib.rs:62-70; stride rules follow
// ug-core/src/cpu_runtime.rs:527-619).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <mutex>

#include "bf16_split.h"
#include "gemm.h"
#include "internal.h"
#include "ughip.h"
#include "wave_ops.h"

using namespace ughip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ floatx16 mma16(const bf16x8& a, const bf16x8& b, const floatx16& c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ floatx16 mma16(const f16x8& a, const f16x8& b, const floatx16& c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }

// MFMA 32x32 accumulator layout: lane l, register i -> row (i/4)*8 + (l/32)*4 + i%4, col l%32.
template <typename T>
__device__ __forceinline__ void store_acc(T* __restrict__ C, const floatx16& acc, int row0, int col, int M, int N, int lane) {
  if (col >= N) return;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    int row = row0 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
    if (row < M) C[(size_t)row * N + col] = (T)acc[i];
  }
}

// ---- any shape, any strides: 64x64 tile per workgroup, one 32x32 MFMA tile per wave ----------------
__global__ void __launch_bounds__(256) gemm_f32_any(MMArgs p) {
  __shared__ float As[64][17];  // [m][k], odd stride: conflict-free column reads
  __shared__ float Bs[16][65];  // [k][n]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const float* __restrict__ A = static_cast<const float*>(p.a) + (size_t)blockIdx.z * p.a_bs;
  const float* __restrict__ B = static_cast<const float*>(p.b) + (size_t)blockIdx.z * p.b_bs;
  float* __restrict__ C = static_cast<float*>(p.c) + (size_t)blockIdx.z * p.c_bs;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  floatx16 acc = {0};
  for (int k0 = 0; k0 < p.K; k0 += 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int e = tid + i * 256, r, k;
      if (p.a_cs == 1) {
        r = e >> 4;
        k = e & 15;
      } else {
        r = e & 63;
        k = e >> 6;
      }
      As[r][k] = (m0 + r < p.M && k0 + k < p.K) ? A[(long long)(m0 + r) * p.a_rs + (long long)(k0 + k) * p.a_cs] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int e = tid + i * 256, k, n;
      if (p.b_cs == 1) {
        k = e >> 6;
        n = e & 63;
      } else {
        k = e & 15;
        n = e >> 4;
      }
      Bs[k][n] = (k0 + k < p.K && n0 + n < p.N) ? B[(long long)(k0 + k) * p.b_rs + (long long)(n0 + n) * p.b_cs] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; kk += 2) {
      float a = As[wm + (lane & 31)][kk + (lane >> 5)];
      float b = Bs[kk + (lane >> 5)][wn + (lane & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  store_acc(C, acc, m0 + wm, n0 + wn + (lane & 31), p.M, p.N, lane);
}

template <typename T>
__global__ void __launch_bounds__(256) gemm_half_any(MMArgs p) {
  typedef T TV __attribute__((ext_vector_type(8)));
  __shared__ __attribute__((aligned(16))) T As[64][40];  // [m][k], 80-byte rows: conflict-free b128 reads
  __shared__ __attribute__((aligned(16))) T Bs[64][40];  // [n][k]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const T* __restrict__ A = static_cast<const T*>(p.a) + (size_t)blockIdx.z * p.a_bs;
  const T* __restrict__ B = static_cast<const T*>(p.b) + (size_t)blockIdx.z * p.b_bs;
  T* __restrict__ C = static_cast<T*>(p.c) + (size_t)blockIdx.z * p.c_bs;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  floatx16 acc = {0};
  for (int k0 = 0; k0 < p.K; k0 += 32) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int e = tid + i * 256, r, k;
      if (p.a_cs == 1) {
        r = e >> 5;
        k = e & 31;
      } else {
        r = e & 63;
        k = e >> 6;
      }
      As[r][k] = (m0 + r < p.M && k0 + k < p.K) ? A[(long long)(m0 + r) * p.a_rs + (long long)(k0 + k) * p.a_cs] : (T)0.f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int e = tid + i * 256, k, n;
      if (p.b_cs == 1) {
        k = e >> 6;
        n = e & 63;
      } else {
        k = e & 31;
        n = e >> 5;
      }
      Bs[n][k] = (k0 + k < p.K && n0 + n < p.N) ? B[(long long)(k0 + k) * p.b_rs + (long long)(n0 + n) * p.b_cs] : (T)0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 32; kk += 16) {
      TV a = *reinterpret_cast<const TV*>(&As[wm + (lane & 31)][kk + (lane >> 5) * 8]);
      TV b = *reinterpret_cast<const TV*>(&Bs[wn + (lane & 31)][kk + (lane >> 5) * 8]);
      acc = mma16(a, b, acc);
    }
    __syncthreads();
  }
  store_acc(C, acc, m0 + wm, n0 + wn + (lane & 31), p.M, p.N, lane);
}

// ---- GEMV kernels for the m <= 8 rows of decode ---------------------------------------------------
// All of them stream the big operand from HBM exactly once with 128-bit loads (x comes from L2),
// accumulate in f32 and reduce in a fixed order, so results do not change from run to run.

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  typedef floatx4 type;
  static constexpr int N = 4;
};
template <>
struct Vec<__bf16> {
  typedef bf16x8 type;
  static constexpr int N = 8;
};
template <>
struct Vec<_Float16> {
  typedef f16x8 type;
  static constexpr int N = 8;
};

template <typename T>
__device__ __forceinline__ float dot_vec(const typename Vec<T>::type& w, const typename Vec<T>::type& x, float acc) {
#pragma unroll
  for (int j = 0; j < Vec<T>::N; ++j) acc += (float)w[j] * (float)x[j];
  return acc;
}

// y[r, n] = sum_k x[r, k] * W[n, k] (rhs stored [n, k]).  KS waves share one column, each walking
// every KS-th 64-lane slab of k with four loads in flight per lane; a workgroup covers 4 / KS
// columns.  Short matrices take KS = 4 so that enough waves are in flight to cover HBM latency.
template <typename T, int R, int KS>
__global__ void __launch_bounds__(256) gemv_nt(MMArgs p) {
  typedef typename Vec<T>::type V;
  constexpr int VE = Vec<T>::N;
  __shared__ float part[4][R];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * (4 / KS) + wave / KS, ks = wave % KS;
  const bool live = n < p.N;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  if (live) {
    const T* __restrict__ X = static_cast<const T*>(p.a) + (size_t)blockIdx.z * p.a_bs;
    const T* __restrict__ W = static_cast<const T*>(p.b) + (size_t)blockIdx.z * p.b_bs + (size_t)n * p.b_cs;
    constexpr int stride = 64 * VE * KS;
    int k = (ks * 64 + lane) * VE;
    for (; k + 3 * stride < p.K; k += 4 * stride) {
      // every matrix element is read once per launch: loads that do not claim cache lines
      const V w0 = __builtin_nontemporal_load(reinterpret_cast<const V*>(W + k)), w1 = __builtin_nontemporal_load(reinterpret_cast<const V*>(W + k + stride));
      const V w2 = __builtin_nontemporal_load(reinterpret_cast<const V*>(W + k + 2 * stride)), w3 = __builtin_nontemporal_load(reinterpret_cast<const V*>(W + k + 3 * stride));
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (r < p.M) {
          const T* Xr = X + (size_t)r * p.a_rs + k;
          acc[r] = dot_vec<T>(w0, *reinterpret_cast<const V*>(Xr), acc[r]);
          acc[r] = dot_vec<T>(w1, *reinterpret_cast<const V*>(Xr + stride), acc[r]);
          acc[r] = dot_vec<T>(w2, *reinterpret_cast<const V*>(Xr + 2 * stride), acc[r]);
          acc[r] = dot_vec<T>(w3, *reinterpret_cast<const V*>(Xr + 3 * stride), acc[r]);
        }
      }
    }
    for (; k < p.K; k += stride) {
      const V w = *reinterpret_cast<const V*>(W + k);
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r < p.M) acc[r] = dot_vec<T>(w, *reinterpret_cast<const V*>(X + (size_t)r * p.a_rs + k), acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
  T* __restrict__ Y = static_cast<T*>(p.c) + (size_t)blockIdx.z * p.c_bs;
  if (KS == 1) {
    if (live && lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r < p.M) Y[(size_t)r * p.N + n] = (T)acc[r];
    }
  } else {
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) part[wave][r] = acc[r];
    }
    __syncthreads();
    if (live && ks == 0 && lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (r < p.M) {
          float s = part[wave][r];
#pragma unroll
          for (int j = 1; j < KS; ++j) s += part[wave + j][r];
          Y[(size_t)r * p.N + n] = (T)s;
        }
      }
    }
  }
}

// Same product for short k (attention scores of one query: k = head size): 16 lanes per column,
// 16 columns per workgroup, no LDS.
template <typename T, int R>
__global__ void __launch_bounds__(256) gemv_nt_short_k(MMArgs p) {
  typedef typename Vec<T>::type V;
  constexpr int VE = Vec<T>::N;
  const int lane = threadIdx.x & 63, sub = lane & 15;
  const int n = blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool live = n < p.N;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  if (live) {
    const T* __restrict__ X = static_cast<const T*>(p.a) + (size_t)blockIdx.z * p.a_bs;
    const T* __restrict__ W = static_cast<const T*>(p.b) + (size_t)blockIdx.z * p.b_bs + (size_t)n * p.b_cs;
    for (int k = sub * VE; k < p.K; k += 16 * VE) {
      const V w = *reinterpret_cast<const V*>(W + k);
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r < p.M) acc[r] = dot_vec<T>(w, *reinterpret_cast<const V*>(X + (size_t)r * p.a_rs + k), acc[r]);
    }
  }
  T* __restrict__ Y = static_cast<T*>(p.c) + (size_t)blockIdx.z * p.c_bs;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float v = acc[r];
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if (live && sub == 0 && r < p.M) Y[(size_t)r * p.N + n] = (T)v;
  }
}

// y[r, n] = sum_k x[r, k] * B[k, n] with B stored [k, n] (attention output of one query: k = the
// sequence).  A workgroup of 1024 threads owns 64 columns: 16 lanes read one 256-byte row segment,
// 64 row slices run in parallel, partial sums meet through LDS.  f32 only, N % 4 == 0.
template <int R>
__global__ void __launch_bounds__(1024) gemv_nn_f32(MMArgs p) {
  __shared__ floatx4 part[16][16][R];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c4 = tid & 15, ksl = tid >> 4;
  const int n = blockIdx.x * 64 + c4 * 4;
  const bool live = n < p.N;
  floatx4 acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = floatx4{0.f, 0.f, 0.f, 0.f};
  if (live) {
    const float* __restrict__ X = static_cast<const float*>(p.a) + (size_t)blockIdx.z * p.a_bs;
    const float* __restrict__ B = static_cast<const float*>(p.b) + (size_t)blockIdx.z * p.b_bs + n;
    int k = ksl;
    for (; k + 192 < p.K; k += 256) {
      const floatx4 b0 = *reinterpret_cast<const floatx4*>(B + (size_t)k * p.b_rs);
      const floatx4 b1 = *reinterpret_cast<const floatx4*>(B + (size_t)(k + 64) * p.b_rs);
      const floatx4 b2 = *reinterpret_cast<const floatx4*>(B + (size_t)(k + 128) * p.b_rs);
      const floatx4 b3 = *reinterpret_cast<const floatx4*>(B + (size_t)(k + 192) * p.b_rs);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (r < p.M) {
          const float* Xr = X + (size_t)r * p.a_rs + k;
          acc[r] += Xr[0] * b0;
          acc[r] += Xr[64] * b1;
          acc[r] += Xr[128] * b2;
          acc[r] += Xr[192] * b3;
        }
      }
    }
    for (; k < p.K; k += 64) {
      const floatx4 b0 = *reinterpret_cast<const floatx4*>(B + (size_t)k * p.b_rs);
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r < p.M) acc[r] += X[(size_t)r * p.a_rs + k] * b0;
    }
  }
  // the 4 row slices of one wave (lanes 16 apart), then the 16 waves in order
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float v = acc[r][c];
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      acc[r][c] = v;
    }
    if (lane < 16) part[wave][lane][r] = acc[r];
  }
  __syncthreads();
  if (tid < 16 && live) {
    float* __restrict__ Y = static_cast<float*>(p.c) + (size_t)blockIdx.z * p.c_bs;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r < p.M) {
        floatx4 s = part[0][tid][r];
#pragma unroll
        for (int w = 1; w < 16; ++w) s += part[w][tid][r];
        *reinterpret_cast<floatx4*>(Y + (size_t)r * p.N + n) = s;
      }
    }
  }
}

template <typename T, int KS>
void launch_gemv_nt(hipStream_t st, const MMArgs& p, size_t b) {
  dim3 grid((unsigned)((p.N + 4 / KS - 1) / (4 / KS)), 1, (unsigned)b);
  if (p.M == 1) gemv_nt<T, 1, KS><<<grid, 256, 0, st>>>(p);
  else if (p.M <= 4) gemv_nt<T, 4, KS><<<grid, 256, 0, st>>>(p);
  else gemv_nt<T, 8, KS><<<grid, 256, 0, st>>>(p);
}

template <typename T>
void launch_gemv_nt_any(hipStream_t st, const MMArgs& p, size_t b) {
  constexpr int VE = Vec<T>::N;
  if (p.K < 64 * VE) {
    dim3 grid((unsigned)((p.N + 15) / 16), 1, (unsigned)b);
    if (p.M == 1) gemv_nt_short_k<T, 1><<<grid, 256, 0, st>>>(p);
    else if (p.M <= 4) gemv_nt_short_k<T, 4><<<grid, 256, 0, st>>>(p);
    else gemv_nt_short_k<T, 8><<<grid, 256, 0, st>>>(p);
    return;
  }
  // enough waves to hide HBM latency: about 8192 over the chip
  const size_t cols = (size_t)p.N * b;
  int ks = cols <= 2048 ? 4 : cols <= 6144 ? 2 : 1;
  if (long long v; tune_get(TUNE_GEMV_KS, &v)) ks = (int)v;  // tuning aid: 1, 2 or 4
  if (ks != 1 && ks != 2 && ks != 4) ks = 1;
  while (ks > 1 && p.K < 64 * VE * ks) ks >>= 1;
  if (ks == 4) launch_gemv_nt<T, 4>(st, p, b);
  else if (ks == 2) launch_gemv_nt<T, 2>(st, p, b);
  else launch_gemv_nt<T, 1>(st, p, b);
}

// Batch stride of one operand: cpu_runtime.rs:527-549 / ug-cuda/src/gemm.rs:59-74.
bool batch_stride(size_t rank, const size_t* dims, const size_t* strides, size_t dflt, long long* out) {
  if (rank == 2) {
    *out = (long long)dflt;
    return true;
  }
  if (rank == 3) {
    *out = (long long)strides[0];
    return true;
  }
  size_t s1 = strides[0], s2 = strides[1];
  if (s1 == s2 * dims[1]) {
    *out = (long long)s2;
    return true;
  }
  if (dims[0] == 1) {
    *out = (long long)s2;
    return true;
  }
  if (dims[1] == 1) {
    *out = (long long)s1;
    return true;
  }
  return false;
}

}  // namespace

// Partial tiles of ughip_matmul_noalloc's split-K products.  Every GPU the library runs on holds its own
// copy of this array at its own address for the life of the process.  In host code the name `scratch` is
// only a handle for hipGetSymbolAddress -- never a device address: kernels, copies and fills get the
// per-device pointer that matmul_scratch_setup() stored in the device.
static __device__ __align__(256) float scratch[UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES / sizeof(float)];

namespace ughip {
// Called once per device from ughip_device_create, with that device current.
int matmul_scratch_setup(ughip_device* dev) {
  void* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) return set_error(UGHIP_ERR_HIP, "hipGetSymbolAddress(matmul scratch) on device %d: %s", dev->ordinal, hipGetErrorString(e));
  dev->static_scratch = ptr;
  return UGHIP_OK;
}
}  // namespace ughip

// The per-device block the split-K partial tiles go to, grown (never shrunk) to `bytes`.
static int grow_gemm_ws(ughip_device* dev, size_t bytes) {
  if (bytes <= dev->gemm_ws_bytes) return UGHIP_OK;
  std::lock_guard<std::mutex> g(dev->mu);
  UGHIP_HIPCHK(hipStreamSynchronize(dev->stream));  // earlier launches may still read the old block
  if (dev->gemm_ws) (void)hipFree(dev->gemm_ws);
  dev->gemm_ws = nullptr;
  dev->gemm_ws_bytes = 0;
  const size_t want = std::max<size_t>(bytes, (size_t)32 << 20);
  UGHIP_HIPCHK(hipMalloc(&dev->gemm_ws, want));
  dev->gemm_ws_bytes = want;
  return UGHIP_OK;
}

// The per-device block for what lies between the launches of one call on rows (normalised rows, the rows between the two
// products of an MLP block); same life cycle.
static int grow_rows_ws(ughip_device* dev, size_t bytes) {
  if (bytes <= dev->rows_ws_bytes) return UGHIP_OK;
  std::lock_guard<std::mutex> g(dev->mu);
  UGHIP_HIPCHK(hipStreamSynchronize(dev->stream));
  if (dev->rows_ws) (void)hipFree(dev->rows_ws);
  dev->rows_ws = nullptr;
  dev->rows_ws_bytes = 0;
  const size_t want = std::max<size_t>(bytes, (size_t)16 << 20);
  UGHIP_HIPCHK(hipMalloc(&dev->rows_ws, want));
  dev->rows_ws_bytes = want;
  return UGHIP_OK;
}

// Which kernel family a product goes to: decided from shapes, strides, offsets and alignment alone, so that the choice can be
// asked for without a device (ughip_matmul_plan) and is the same one the launch makes.
enum Route { ROUTE_GEMV_NT, ROUTE_GEMV_NN, ROUTE_DMA, ROUTE_DMA_F32, ROUTE_X6, ROUTE_TILED, ROUTE_ANY, ROUTE_UNSUPPORTED };

__global__ void split3_operands_kernel(const float* __restrict__ xa, uint16_t* __restrict__ pa, size_t na4, int ka, unsigned a_blocks, const float* __restrict__ xb,
                                       uint16_t* __restrict__ pb, size_t nb4, int bk, int b_kn);  // defined with the products of rows below

// An f32 product as six bf16 terms (UGHIP_MATMUL_X6=1; never the default: the f32 product's accuracy, not its bits): the
// problem as the 16-bit kernel sees it once both operands are split into three bf16 planes per 64 elements of k -- rows of
// 3 k elements, a loop over 6 k -- and the tile it takes it with (0: not this product's route).  Contiguous operands, either
// rhs layout, k % 64 == 0, n % 8 == 0.  The pointers of the result are stand-ins until the planes exist.
static int matmul_x6_plan(const MMArgs& p, size_t b, size_t lhs_offset, size_t rhs_offset, MMArgs* out) {
  long long on = 0;
  if (!tune_get(TUNE_MATMUL_X6, &on) || !on) return 0;
  const long long m = p.M, n = p.N, k = p.K;
  if (m < 9 || k % 64 != 0 || n % 8 != 0 || k > 0x7fffffffll / 6) return 0;
  if (p.a_cs != 1 || p.a_rs != k || (b > 1 && p.a_bs != m * k) || lhs_offset % 4 != 0 || rhs_offset % 4 != 0) return 0;
  const bool nn = p.b_cs == 1 && p.b_rs == n && n != 1, nt = p.b_rs == 1 && p.b_cs == k;
  if (nn == nt || (b > 1 && p.b_bs != n * k)) return 0;
  if ((reinterpret_cast<uintptr_t>(p.a) | reinterpret_cast<uintptr_t>(p.b) | reinterpret_cast<uintptr_t>(p.c)) & 15) return 0;
  MMArgs q = p;
  q.K = (int)(6 * k);
  q.a_rs = 3 * k, q.a_cs = 1, q.a_bs = m * 3 * k;
  if (nn) q.b_rs = n, q.b_cs = 1;
  else q.b_rs = 1, q.b_cs = 3 * k;
  q.b_bs = n * 3 * k;
  q.a = q.b = reinterpret_cast<const void*>(uintptr_t(1) << 20);
  int best = 0;
  double best_us = 0;
  for (int tile : {256, 128, 64}) {
    if (!gemm_dma_planes6_supported(q, b, tile)) continue;
    const double us = gemm_dma_cost_us(q, b, tile);
    if (!best || us < best_us * 0.97) best = tile, best_us = us;
  }
  if (best && out) *out = q;
  return best;
}
static Route matmul_route(int dtype, bool mixed, const MMArgs& p, size_t b, size_t lhs_offset, size_t rhs_offset, int* dma_tile, bool allow_x6 = true) {
  const size_t m = (size_t)p.M, n = (size_t)p.N, k = (size_t)p.K;
  const bool f32 = dtype == UGHIP_F32;
  const size_t vec = f32 ? 4 : 8;
  // m <= 8: GEMV kernels.  Vector loads need 16-byte aligned rows; strides of size-1 dims are never used.
  const long long lv = (long long)vec;
  const bool small_m = m <= 8 && p.a_cs == 1 && b <= 65535;
  const bool lhs_vec_ok = (m == 1 || p.a_rs % lv == 0) && (b == 1 || p.a_bs % lv == 0) && lhs_offset % vec == 0;
  const bool rhs_vec_ok = (b == 1 || p.b_bs % lv == 0) && rhs_offset % vec == 0;
  const bool gemv_nt_ok = small_m && lhs_vec_ok && rhs_vec_ok && k % vec == 0 && p.b_rs == 1 && (n == 1 || p.b_cs % lv == 0);
  const bool gemv_nn_ok = small_m && f32 && rhs_vec_ok && n % 4 == 0 && p.b_cs == 1 && (k == 1 || p.b_rs % 4 == 0);
  if (mixed && (!gemm_tiled_supported(UGHIP_F32, p, b, true) || rhs_offset % 8 != 0)) return ROUTE_UNSUPPORTED;
  if (!mixed && gemv_nt_ok) return ROUTE_GEMV_NT;
  if (!mixed && gemv_nn_ok) return ROUTE_GEMV_NN;
  if (const int bn = mixed ? 0 : gemm_dma_pick(dtype, p, b)) {
    *dma_tile = bn;
    return ROUTE_DMA;
  }
  if (f32 && !mixed && allow_x6)
    if (const int tile = matmul_x6_plan(p, b, lhs_offset, rhs_offset, nullptr)) {
      *dma_tile = tile;
      return ROUTE_X6;
    }
  if (f32 && !mixed && gemm_dma_f32_pick(p, b)) return ROUTE_DMA_F32;
  return gemm_tiled_supported(dtype, p, b, mixed) ? ROUTE_TILED : ROUTE_ANY;
}

static int matmul_impl(ughip_device* dev, ughip_slice* dst, const ughip_slice* lhs, const ughip_slice* rhs, size_t b, size_t m, size_t n, size_t k,
                       size_t rank, const size_t* lhs_dims, const size_t* lhs_strides, size_t lhs_offset, const size_t* rhs_dims, const size_t* rhs_strides,
                       size_t rhs_offset, bool no_alloc) {
  if (!dev || !dst || !lhs || !rhs) return set_error(UGHIP_ERR_INVALID, "matmul: null argument");
  if (rank < 2 || rank > 4 || !lhs_dims || !lhs_strides || !rhs_dims || !rhs_strides)
    return set_error(UGHIP_ERR_INVALID, "matmul: rank %zu layouts are not supported", rank);
  // One dtype for all three (lib.rs:62-70), with one addition: an F32 product may read a BF16 rhs (weights
  // kept as a checkpoint stores them); it is widened on the way in, which is exact.
  const bool mixed = dst->dtype == UGHIP_F32 && lhs->dtype == UGHIP_F32 && rhs->dtype == UGHIP_BF16;
  if (!mixed && (dst->dtype != lhs->dtype || dst->dtype != rhs->dtype || (dst->dtype != UGHIP_F32 && dst->dtype != UGHIP_BF16 && dst->dtype != UGHIP_F16))) {
    int code = (dst->dtype == lhs->dtype && dst->dtype == rhs->dtype) ? UGHIP_ERR_UNSUPPORTED : UGHIP_ERR_INVALID;
    return set_error(code, "incorrect dtypes for matmul, dst: %s, lhs: %s, rhs: %s", dtype_name(dst->dtype), dtype_name(lhs->dtype),
                     dtype_name(rhs->dtype));
  }
  if (dst == lhs || dst == rhs) return set_error(UGHIP_ERR_INVALID, "matmul: dst aliases an operand (already borrowed)");
  if (b > 65535 || m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "matmul: shape too large");
  MMArgs p;
  p.M = (int)m;
  p.N = (int)n;
  p.K = (int)k;
  p.a_rs = (long long)lhs_strides[rank - 2];
  p.a_cs = (long long)lhs_strides[rank - 1];
  p.b_rs = (long long)rhs_strides[rank - 2];
  p.b_cs = (long long)rhs_strides[rank - 1];
  if (!batch_stride(rank, lhs_dims, lhs_strides, m * k, &p.a_bs)) return set_error(UGHIP_ERR_STRIDING, "matmul: non-contiguous lhs batch strides");
  if (!batch_stride(rank, rhs_dims, rhs_strides, n * k, &p.b_bs)) return set_error(UGHIP_ERR_STRIDING, "matmul: non-contiguous rhs batch strides");
  p.c_bs = (long long)(m * n);
  if (dst->len < b * m * n) return set_error(UGHIP_ERR_BOUNDS, "matmul: dst has %zu elements, needs %zu", dst->len, b * m * n);
  if (b == 0 || m == 0 || n == 0) return UGHIP_OK;
  // Furthest element each operand can touch.
  size_t a_max = lhs_offset + (b - 1) * (size_t)p.a_bs + (m - 1) * (size_t)p.a_rs + (k ? (k - 1) * (size_t)p.a_cs : 0);
  size_t b_max = rhs_offset + (b - 1) * (size_t)p.b_bs + (n - 1) * (size_t)p.b_cs + (k ? (k - 1) * (size_t)p.b_rs : 0);
  if (k && (a_max >= lhs->len || b_max >= rhs->len))
    return set_error(UGHIP_ERR_BOUNDS, "matmul: operand too short for its layout (lhs %zu/%zu, rhs %zu/%zu)", a_max, lhs->len, b_max, rhs->len);
  if (int rc = device_activate(dev)) return rc;
  const size_t esz = dst->dtype == UGHIP_F32 ? 4 : 2;
  p.a = static_cast<const char*>(lhs->ptr) + lhs_offset * esz;
  p.b = static_cast<const char*>(rhs->ptr) + rhs_offset * (mixed ? 2 : esz);
  p.c = dst->ptr;
  const bool f32 = dst->dtype == UGHIP_F32;
  hipStream_t st = dev->stream;
  int dma_tile = 0;
  const Route route = matmul_route(dst->dtype, mixed, p, b, lhs_offset, rhs_offset, &dma_tile, !no_alloc);
  const bool gemv_nt_ok = route == ROUTE_GEMV_NT, gemv_nn_ok = route == ROUTE_GEMV_NN;
  if (route == ROUTE_UNSUPPORTED)
    return set_error(UGHIP_ERR_UNSUPPORTED,
                     "matmul: an F32 product with a BF16 rhs is built for an [n, k]-major rhs with k a multiple of 32 and rows that "
                     "start on 8-byte boundaries (got m %zu, n %zu, k %zu, rhs strides %lld, %lld)",
                     m, n, k, p.b_rs, p.b_cs);
  const char* tn = f32 ? "f32" : dst->dtype == UGHIP_F16 ? "f16" : "bf16";
  if (!mixed && gemv_nt_ok) {
    note_kernel("gemv_nt<%s>", tn);
    if (f32) launch_gemv_nt_any<float>(st, p, b);
    else if (dst->dtype == UGHIP_F16) launch_gemv_nt_any<_Float16>(st, p, b);
    else launch_gemv_nt_any<__bf16>(st, p, b);
  } else if (!mixed && gemv_nn_ok) {
    note_kernel("gemv_nn<f32>");
    dim3 grid((unsigned)((n + 63) / 64), 1, (unsigned)b);
    if (m == 1) gemv_nn_f32<1><<<grid, 1024, 0, st>>>(p);
    else if (m <= 4) gemv_nn_f32<4><<<grid, 1024, 0, st>>>(p);
    else gemv_nn_f32<8><<<grid, 1024, 0, st>>>(p);
  } else if (route == ROUTE_DMA) {
    UGHIP_HIPCHK(gemm_dma_launch(st, dst->dtype, p, b, dma_tile));
    return UGHIP_OK;
  } else if (route == ROUTE_DMA_F32) {
    UGHIP_HIPCHK(gemm_dma_f32_launch(st, p, b));
    return UGHIP_OK;
  } else if (route == ROUTE_X6) {
    MMArgs q;
    if (matmul_x6_plan(p, b, lhs_offset, rhs_offset, &q) != dma_tile) return set_error(UGHIP_ERR_HIP, "matmul: the six-term plan changed between its two readings");
    // [planes of the lhs | planes of the rhs] in the scratch block, 6 bytes an element
    const size_t a_elems = b * m * k, b_elems = b * n * k, a_bytes = (a_elems * 6 + 255) & ~(size_t)255;
    if (int rc = grow_gemm_ws(dev, a_bytes + b_elems * 6)) return rc;
    uint16_t* ap = static_cast<uint16_t*>(dev->gemm_ws);
    uint16_t* bp = reinterpret_cast<uint16_t*>(static_cast<char*>(dev->gemm_ws) + a_bytes);
    const size_t a_blocks = (a_elems / 4 + 255) / 256, b_blocks = (b_elems / 4 + 255) / 256;
    if (a_blocks + b_blocks > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "matmul: operands too large for the pass that splits them");
    const bool b_kn = q.b_cs == 1;
    split3_operands_kernel<<<(unsigned)(a_blocks + b_blocks), 256, 0, st>>>(static_cast<const float*>(p.a), ap, a_elems / 4, (int)k, (unsigned)a_blocks,
                                                                           static_cast<const float*>(p.b), bp, b_elems / 4, (int)(b_kn ? n : k), b_kn ? 1 : 0);
    UGHIP_HIPCHK(hipGetLastError());
    q.a = ap, q.b = bp, q.c = dst->ptr;
    UGHIP_HIPCHK(gemm_dma_launch_planes6(st, q, b, dma_tile));
    return UGHIP_OK;
  } else if (route == ROUTE_TILED) {
    const size_t ws_bytes = gemm_tiled_workspace_bytes(dst->dtype, p, b);
    if (no_alloc) {
      // the partial tiles go to the device's copy of the static array; every slab writes its whole tile before
      // the fold reads it, so nothing has to be cleared between calls
      if (ws_bytes > (size_t)UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES)
        return set_error(UGHIP_ERR_UNSUPPORTED,
                         "matmul_noalloc: this product splits K and needs %zu bytes for its partial tiles, the static scratch holds %zu "
                         "(b %zu, m %zu, n %zu, k %zu); use ughip_matmul",
                         ws_bytes, (size_t)UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES, b, m, n, k);
      if (ws_bytes && !dev->static_scratch) return set_error(UGHIP_ERR_HIP, "matmul_noalloc: the static scratch of device %d was not set up", dev->ordinal);
      UGHIP_HIPCHK(gemm_tiled_launch(st, dst->dtype, p, b, ws_bytes ? static_cast<float*>(dev->static_scratch) : nullptr, mixed));
      return UGHIP_OK;
    }
    if (int rc = grow_gemm_ws(dev, ws_bytes)) return rc;
    UGHIP_HIPCHK(gemm_tiled_launch(st, dst->dtype, p, b, ws_bytes ? static_cast<float*>(dev->gemm_ws) : nullptr, mixed));
    return UGHIP_OK;
  } else {
    dim3 grid((unsigned)((n + 63) / 64), (unsigned)((m + 63) / 64), (unsigned)b);
    if (grid.y > 65535 || b > 65535) return set_error(UGHIP_ERR_INVALID, "matmul: m or batch too large for this kernel");
    note_kernel("gemm_any<%s>", tn);
    if (f32) gemm_f32_any<<<grid, 256, 0, st>>>(p);
    else if (dst->dtype == UGHIP_F16) gemm_half_any<_Float16><<<grid, 256, 0, st>>>(p);
    else gemm_half_any<__bf16><<<grid, 256, 0, st>>>(p);
  }
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

extern "C" int ughip_matmul(ughip_device* dev, ughip_slice* dst, const ughip_slice* lhs, const ughip_slice* rhs, size_t b, size_t m, size_t n,
                            size_t k, size_t rank, const size_t* lhs_dims, const size_t* lhs_strides, size_t lhs_offset, const size_t* rhs_dims,
                            const size_t* rhs_strides, size_t rhs_offset) {
  return matmul_impl(dev, dst, lhs, rhs, b, m, n, k, rank, lhs_dims, lhs_strides, lhs_offset, rhs_dims, rhs_strides, rhs_offset, false);
}

extern "C" int ughip_matmul_noalloc(ughip_device* dev, ughip_slice* dst, const ughip_slice* lhs, const ughip_slice* rhs, size_t b, size_t m, size_t n,
                                    size_t k, size_t rank, const size_t* lhs_dims, const size_t* lhs_strides, size_t lhs_offset,
                                    const size_t* rhs_dims, const size_t* rhs_strides, size_t rhs_offset) {
  return matmul_impl(dev, dst, lhs, rhs, b, m, n, k, rank, lhs_dims, lhs_strides, lhs_offset, rhs_dims, rhs_strides, rhs_offset, true);
}

__global__ void __launch_bounds__(256) split3_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ x3, size_t n4, int k) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  const size_t e = g * 4, row = e / (size_t)k, col = e % (size_t)k;
  const float4 v = reinterpret_cast<const float4*>(x)[g];
  const float in[4] = {v.x, v.y, v.z, v.w};
  split3_store4(in, x3 + row * 3 * (size_t)k, col);
}

// RMSNorm of the rows of x [m, k] (model.rs:65-78: x / sqrt(mean(x^2) + eps) * alpha, the division as a multiplication by
// the reciprocal, like the single-row projections do), one workgroup per row; the row's second pass comes from cache.
// PLANES: the normalised row goes out as its three bf16 planes (what split3_bf16_kernel would make of it), else as f32.
// An operand stored [k, n] (k % 64 == 0) is split the same way with the planes of rows kk .. kk + 63 as rows 3 kk .. of the
// result: 64 rows of first terms, then 64 of second, then 64 of third ones (every batch element a multiple of 64 rows).
// Both operands of a product in one launch: blocks 0 .. a_blocks - 1 split the lhs like split3_bf16_kernel, the rest the rhs,
// like split3_bf16_kernel ([n, k]-major: b_kn == 0, bk = k) or by rows as described above ([k, n]-major: bk = n).
__global__ void __launch_bounds__(256) split3_operands_kernel(const float* __restrict__ xa, uint16_t* __restrict__ pa, size_t na4, int ka, unsigned a_blocks,
                                                              const float* __restrict__ xb, uint16_t* __restrict__ pb, size_t nb4, int bk, int b_kn) {
  const bool lhs = blockIdx.x < a_blocks;
  const size_t g = (size_t)(lhs ? blockIdx.x : blockIdx.x - a_blocks) * 256 + threadIdx.x;
  if (g >= (lhs ? na4 : nb4)) return;
  const float* __restrict__ x = lhs ? xa : xb;
  uint16_t* __restrict__ x3 = lhs ? pa : pb;
  const size_t w = (size_t)(lhs ? ka : bk), e = g * 4, row = e / w, col = e % w;
  const float4 v = reinterpret_cast<const float4*>(x)[g];
  const float in[4] = {v.x, v.y, v.z, v.w};
  if (lhs || !b_kn) {
    split3_store4(in, x3 + row * 3 * w, col);
  } else {
    uint16_t hi[4], mid[4], lo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) split3(in[i], hi[i], mid[i], lo[i]);
    uint16_t* o = x3 + ((row / 64) * 192 + row % 64) * w + col;
    *reinterpret_cast<ushort4*>(o) = make_ushort4(hi[0], hi[1], hi[2], hi[3]);
    *reinterpret_cast<ushort4*>(o + 64 * w) = make_ushort4(mid[0], mid[1], mid[2], mid[3]);
    *reinterpret_cast<ushort4*>(o + 128 * w) = make_ushort4(lo[0], lo[1], lo[2], lo[3]);
  }
}

// NV: 16-byte groups a thread keeps of its row between the two passes (k <= 1024 NV; the row and alpha are requested at
// once, and only the reduction lies between the loads and the stores); 0: any k, the second pass reads the row again.
template <bool PLANES, int NV>
__global__ void __launch_bounds__(256) rms_norm_rows_kernel(const float* __restrict__ x, const float* __restrict__ alpha, float eps, void* __restrict__ out, int k) {
  __shared__ float part[4];
  const size_t row = blockIdx.x;
  const float4* __restrict__ xr = reinterpret_cast<const float4*>(x + row * (size_t)k);
  const float4* __restrict__ ar = reinterpret_cast<const float4*>(alpha);
  const int k4 = k / 4, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float4 v[NV ? NV : 1], a[NV ? NV : 1];
  float ss = 0.f;
  if (NV) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = j * 256 + (int)threadIdx.x;
      v[j] = i < k4 ? xr[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      a[j] = i < k4 ? ar[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      ss += v[j].x * v[j].x;
      ss += v[j].y * v[j].y;
      ss += v[j].z * v[j].z;
      ss += v[j].w * v[j].w;
    }
  } else {
    for (int i = threadIdx.x; i < k4; i += 256) {
      const float4 t = xr[i];
      ss += t.x * t.x;
      ss += t.y * t.y;
      ss += t.z * t.z;
      ss += t.w * t.w;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  if (lane == 0) part[wave] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const float inv = 1.f / sqrtf(ss * (1.f / (float)k) + eps);
  auto put = [&](int i, const float4& t, const float4& al) {
    const float y[4] = {t.x * inv * al.x, t.y * inv * al.y, t.z * inv * al.z, t.w * inv * al.w};
    if (PLANES) split3_store4(y, static_cast<uint16_t*>(out) + row * 3 * (size_t)k, (size_t)i * 4);
    else reinterpret_cast<float4*>(static_cast<float*>(out) + row * (size_t)k)[i] = make_float4(y[0], y[1], y[2], y[3]);
  };
  if (NV) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = j * 256 + (int)threadIdx.x;
      if (i < k4) put(i, v[j], a[j]);
    }
  } else {
    for (int i = threadIdx.x; i < k4; i += 256) put(i, xr[i], ar[i]);
  }
}
template <bool PLANES>
static hipError_t rms_norm_rows_launch(hipStream_t stream, const float* x, const float* alpha, float eps, void* out, size_t m, size_t k) {
  const dim3 grid((unsigned)m), block(256);
  if (k <= 2048) rms_norm_rows_kernel<PLANES, 2><<<grid, block, 0, stream>>>(x, alpha, eps, out, (int)k);
  else if (k <= 4096) rms_norm_rows_kernel<PLANES, 4><<<grid, block, 0, stream>>>(x, alpha, eps, out, (int)k);
  else rms_norm_rows_kernel<PLANES, 0><<<grid, block, 0, stream>>>(x, alpha, eps, out, (int)k);
  return hipGetLastError();
}

// The fold of a stacked gate | up product (gemm_split_reduce with SwiGLU: the slabs added in index order, then
// silu(gate) * up) whose result goes out as the three bf16 planes of rows of n / 2 elements instead of f32: what the
// product behind it (down) reads, without the f32 rows in between and the pass that splits them.
__global__ void __launch_bounds__(256) swiglu_fold_planes_kernel(const float* __restrict__ ws, uint16_t* __restrict__ x3, size_t n4, size_t slab_elems, int nsplit, int n) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const size_t half4 = (size_t)n / 8, r = g / half4, j4 = g % half4;
  const size_t gate = r * ((size_t)n / 4) + j4, up = gate + half4;
  f32x4 a = reinterpret_cast<const f32x4*>(ws)[gate], b = reinterpret_cast<const f32x4*>(ws)[up];
  for (int k = 1; k < nsplit; ++k) {
    a += reinterpret_cast<const f32x4*>(ws + (size_t)k * slab_elems)[gate];
    b += reinterpret_cast<const f32x4*>(ws + (size_t)k * slab_elems)[up];
  }
  const float y[4] = {a.x / (1.f + expf(-a.x)) * b.x, a.y / (1.f + expf(-a.y)) * b.y, a.z / (1.f + expf(-a.z)) * b.z, a.w / (1.f + expf(-a.w)) * b.w};
  split3_store4(y, x3 + r * 3 * ((size_t)n / 2), j4 * 4);
}

// Which kernel a product of rows takes: decided from shapes, alignment and the cost models alone, so that ughip_linear_rows_plan
// can answer without a device.
struct RowsRoute {
  enum Kind { X3_ROWS, DMA_PLANES, TILED } kind = TILED;
  RowsX3Plan x3;                    // X3_ROWS
  int dma_tile = 0, dma_split = 1;  // DMA_PLANES
};
static RowsRoute rows_route(const MMArgs& p, int dtype, bool x3, GemmEpilogue::Kind kind, const void* x, const void* w, const void* dst, const void* residual, size_t m,
                            size_t rows, size_t k, int num_cus) {
  RowsRoute r;
  // 33 .. 128 rows: the kernel that splits the rows itself (no planes through memory, no launch for the split).  In a 22-layer
  // prefill of 128 positions, with the matrices coming from memory: q|k|v 13.4 us against 17.9 (split + product), o 12.6 against
  // 19.5, gate|up 30.6 against 37.2, down 19.7 against 26.5.  Two row tiles (129 .. 256 rows) were slower than the kernels below,
  // and up to 32 rows its 128-row tile is mostly padding.
  long long x3_rows = -1;
  tune_get(TUNE_X3_ROWS, &x3_rows);
  if (x3 && m > 32 && m <= 128 && x3_rows != 0 && rows_x3_supported(x, w, dst, residual, m, rows, k)) {
    r.kind = RowsRoute::X3_ROWS;
    r.x3 = rows_x3_plan(m, rows, k, x3_rows > 0 ? (int)x3_rows : 0, num_cus);
    return r;
  }
  // Many rows of planes: the one-wave-per-SIMD kernel where it is priced cheaper (a prompt of a thousand positions and
  // more).  Its result leaves as f32 with the residual added on the way; SwiGLU goes through the scratch block and the fold.
  // (from 384 rows: at 128 and 256 rows the register-staged kernel is as fast or faster for four of the five products of a
  // llama step -- q|k|v 25.2 us against 28.6 at 256 rows -- and the model below does not see that; at 512 rows this kernel is)
  long long x3_dma = -1, x3_split = 0;  // tuning aids: X3_DMA 0 keeps the register-staged kernel, 3 / 4 / 5 force a tile; X3_SPLIT n a K split
  tune_get(TUNE_X3_DMA, &x3_dma);
  tune_get(TUNE_X3_SPLIT, &x3_split);
  if (x3 && m >= 384 && x3_dma != 0) {
    MMArgs q = p;
    q.c = const_cast<void*>(dst);  // alignment of the result as f32
    double best = 0;
    const int forced_tile = x3_dma == 3 ? 256 : x3_dma == 4 ? 128 : x3_dma == 5 ? 64 : 0;
    const int forced_split = (int)x3_split;
    for (int tile : {256, 128, 64}) {
      if (forced_tile && tile != forced_tile) continue;
      for (int split : {1, 2, 4, 8}) {
        if (forced_split && split != forced_split) continue;
        if (!gemm_dma_planes3_split_ok(q, split)) continue;
        MMArgs qs = q;
        if (split > 1) qs.K = q.K / split, qs.a_bs = qs.K, qs.b_bs = qs.K / 3, qs.c_bs = (long long)(m * rows);
        if (!gemm_dma_supported(UGHIP_BF16, qs, (size_t)split, tile)) continue;
        // the kernel (its model counts 2 bytes per result element), the f32 result's other 2, and the fold where there is one:
        // the slabs in, the result out, a launch
        const bool fold = split > 1 || kind == GemmEpilogue::SWIGLU;
        const double us = gemm_dma_cost_us(qs, (size_t)split, tile) + (double)split * m * rows * 2 / 6.4e6 + (fold ? 3.0 + (double)(split + 1) * m * rows * 4 / 6.4e6 : 0.0);
        if (!r.dma_tile || us < best * 0.97) r.dma_tile = tile, r.dma_split = split, best = us;
      }
    }
    const double other = gemm_tiled_cost_us(dtype, p, 1);
    if (r.dma_tile && !forced_tile && other >= 0 && other < best * 1.05) r.dma_tile = 0;  // it has to be clearly cheaper: its model is the rougher one
  }
  if (r.dma_tile) r.kind = RowsRoute::DMA_PLANES;
  return r;
}
static const char* dma_planes_tail(GemmEpilogue::Kind kind, bool fold, bool residual) {
  if (!fold) return residual ? ",+residual" : "";
  return kind == GemmEpilogue::SWIGLU ? ",swiglu fold" : kind == GemmEpilogue::ADD ? ",+residual in the fold" : ",fold";
}

// What a product of rows does around itself besides `kind`.
struct RowsAround {
  const float* alpha = nullptr;  // the rows are RMS-normalised first (x / sqrt(mean(x^2) + eps) * alpha) ...
  float eps = 0.f;
  float* xn = nullptr;                  // ... into these m * k floats, unless the pass that writes the planes does it on its way
  const uint16_t* planes_in = nullptr;  // three-term product: the planes of x, already made (x is not read)
  uint16_t* planes_out = nullptr;       // SwiGLU on a route that folds slabs: the result may go here as planes instead of to dst ...
  bool wrote_planes = false;            // ... and this says whether it did
};

static MMArgs rows_args(const void* x, const void* w, void* dst, size_t m, size_t rows, size_t k, bool x3) {
  MMArgs p;
  p.M = (int)m, p.N = (int)rows, p.K = (int)(x3 ? 3 * k : k);
  p.a_rs = (long long)(x3 ? 3 * k : k), p.a_cs = 1, p.b_rs = 1, p.b_cs = (long long)k;
  p.a_bs = (long long)(m * (x3 ? 3 * k : k)), p.b_bs = (long long)(rows * k), p.c_bs = (long long)(m * rows);
  p.a = x, p.b = w, p.c = dst;
  if (x3) p.b_k_div = 3;
  return p;
}

// x [m, k] f32 against a row-major [rows, k] matrix (f32 or bf16) through the tiled kernel, the fold applying `kind`.
// product == UGHIP_PRODUCT_BF16X3 (bf16 matrix): the rows are split into three bf16 planes first and the product runs on
// the bf16 matrix pipe over a K of 3 k, every K tile of the matrix meeting the three planes of its columns in turn.
// Buffers are checked by the callers; x, residual and dst are device pointers to f32.
static int linear_rows_core(ughip_device* dev, const char* what, const float* x, const ughip_slice* w, const float* residual, float* dst, size_t m, size_t rows,
                            size_t k, GemmEpilogue::Kind kind, int product, RowsAround* ar) {
  if (product != UGHIP_PRODUCT_F32 && product != UGHIP_PRODUCT_BF16X3) return set_error(UGHIP_ERR_INVALID, "%s: unknown product %d", what, product);
  if (product == UGHIP_PRODUCT_BF16X3 && w->dtype != UGHIP_BF16)
    return set_error(UGHIP_ERR_INVALID, "%s: the three-term bf16 product needs a BF16 matrix (an F32 one would have to be split as well), got %s", what, dtype_name(w->dtype));
  if (m > 0x7fffffffull || rows > 0x7fffffffull || k > 0x7fffffffull / 3) return set_error(UGHIP_ERR_INVALID, "%s: shape too large", what);
  const size_t out_cols = kind == GemmEpilogue::SWIGLU ? rows / 2 : rows;
  if (m == 0 || rows == 0) return UGHIP_OK;
  const bool x3 = product == UGHIP_PRODUCT_BF16X3;
  const bool norm = ar && ar->alpha, planes_in = ar && ar->planes_in;
  if (planes_in && (!x3 || norm)) return set_error(UGHIP_ERR_INVALID, "%s: planes stand for the rows of a three-term product as they are", what);
  if (norm && (k % 4 != 0 || (reinterpret_cast<uintptr_t>(ar->alpha) & 15))) return set_error(UGHIP_ERR_UNSUPPORTED, "%s: the norm reads 16 bytes at a time (k %zu)", what, k);
  // (x3: p.a is checked for alignment below with the f32 rows standing in; the planes live in 256-byte aligned scratch blocks)
  const void* x_stand_in = planes_in ? static_cast<const void*>(ar->planes_in) : static_cast<const void*>(x);
  MMArgs p = rows_args(x_stand_in, w->ptr, dst, m, rows, k, x3);
  const bool mixed = !x3 && w->dtype == UGHIP_BF16;
  const int dtype = x3 ? UGHIP_BF16 : UGHIP_F32;
  // an F32 matrix under 2 .. 8 rows is the row-vector kernels' job (ughip_matmul); those do not read a BF16 matrix
  const size_t min_rows = w->dtype == UGHIP_BF16 ? 2 : 9;
  if (m < min_rows || rows % 8 != 0 || (kind == GemmEpilogue::SWIGLU && rows % 16 != 0) || (x3 && k % 64 != 0) || !gemm_tiled_supported(dtype, p, 1, mixed))
    return set_error(UGHIP_ERR_UNSUPPORTED, "%s: built for m >= 9 rows (m >= 2 with a BF16 matrix), k %% 32 == 0 (k %% 64 == 0 for the three-term bf16 product), n %% 8 == 0 and 16-byte aligned buffers (got m %zu, n %zu, k %zu)",
                     what, m, out_cols, k);
  if (int rc = device_activate(dev)) return rc;
  GemmEpilogue epi{kind, residual};
  epi.out_f32 = x3;
  const RowsRoute route = rows_route(p, dtype, x3, kind, x_stand_in, w->ptr, dst, residual, m, rows, k, dev->num_cus);
  if (route.kind == RowsRoute::X3_ROWS) {
    if (planes_in) return set_error(UGHIP_ERR_INVALID, "%s: this product splits its rows itself", what);
    if (norm) {
      UGHIP_HIPCHK(rms_norm_rows_launch<false>(dev->stream, x, ar->alpha, ar->eps, ar->xn, m, k));
      x = ar->xn;
    }
    if (int rc = grow_gemm_ws(dev, route.x3.ws_bytes)) return rc;
    UGHIP_HIPCHK(rows_x3_launch(dev->stream, x, w->ptr, static_cast<float*>(dev->gemm_ws), dst, m, rows, k, route.x3, kind, epi.residual));
    return UGHIP_OK;
  }
  const int dma_tile = route.dma_tile, dma_split = route.dma_split;
  const bool dma_fold = dma_tile && (dma_split > 1 || kind == GemmEpilogue::SWIGLU);
  const size_t ws_bytes = dma_tile ? (dma_fold ? ((size_t)dma_split * m * rows * sizeof(float) + 255) & ~(size_t)255 : 0)
                                   : (gemm_tiled_workspace_bytes(dtype, p, 1, &epi) + 255) & ~(size_t)255;
  const size_t x3_bytes = x3 && !planes_in ? m * 3 * k * sizeof(uint16_t) : 0;
  if (int rc = grow_gemm_ws(dev, ws_bytes + x3_bytes)) return rc;
  if (planes_in) {
    p.a = ar->planes_in;
  } else if (x3) {
    uint16_t* planes = reinterpret_cast<uint16_t*>(static_cast<char*>(dev->gemm_ws) + ws_bytes);
    const size_t n4 = m * k / 4;
    if (norm) UGHIP_HIPCHK(rms_norm_rows_launch<true>(dev->stream, x, ar->alpha, ar->eps, planes, m, k));
    else split3_bf16_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, dev->stream>>>(x, planes, n4, (int)k);
    UGHIP_HIPCHK(hipGetLastError());
    p.a = planes;
  } else if (norm) {
    UGHIP_HIPCHK(rms_norm_rows_launch<false>(dev->stream, x, ar->alpha, ar->eps, ar->xn, m, k));
    p.a = ar->xn;
  }
  if (dma_tile) {
    if (dma_fold) {
      p.c = dev->gemm_ws;
      const bool to_planes = kind == GemmEpilogue::SWIGLU && ar && ar->planes_out && out_cols % 64 == 0;
      UGHIP_HIPCHK(gemm_dma_launch_planes3(dev->stream, p, dma_tile, dma_split, nullptr, to_planes ? ",swiglu fold onto planes" : dma_planes_tail(kind, true, false)));
      if (to_planes) {
        const size_t elems = m * rows, n4 = elems / 8;
        swiglu_fold_planes_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, dev->stream>>>(static_cast<const float*>(dev->gemm_ws), ar->planes_out, n4, elems, dma_split, (int)rows);
        UGHIP_HIPCHK(hipGetLastError());
        ar->wrote_planes = true;
      } else {
        UGHIP_HIPCHK(gemm_fold_f32(dev->stream, static_cast<const float*>(dev->gemm_ws), dst, m, rows, dma_split, kind, epi.residual));
      }
    } else {
      UGHIP_HIPCHK(gemm_dma_launch_planes3(dev->stream, p, dma_tile, 1, epi.residual, dma_planes_tail(kind, false, epi.residual != nullptr)));
    }
    return UGHIP_OK;
  }
  UGHIP_HIPCHK(gemm_tiled_launch(dev->stream, dtype, p, 1, static_cast<float*>(dev->gemm_ws), mixed, &epi));
  return UGHIP_OK;
}

static int linear_rows(ughip_device* dev, const char* what, const ughip_slice* x, const ughip_slice* w, const ughip_slice* residual, ughip_slice* dst, size_t m,
                       size_t rows, size_t k, GemmEpilogue::Kind kind, int product, const ughip_slice* alpha = nullptr, float eps = 0.f) {
  if (!dev || !x || !w || !dst || (kind == GemmEpilogue::ADD && !residual)) return set_error(UGHIP_ERR_INVALID, "%s: null argument", what);
  if (x->dtype != UGHIP_F32 || dst->dtype != UGHIP_F32 || (residual && residual->dtype != UGHIP_F32) || (w->dtype != UGHIP_F32 && w->dtype != UGHIP_BF16) ||
      (alpha && alpha->dtype != UGHIP_F32))
    return set_error(UGHIP_ERR_INVALID, "%s: x, residual, alpha and dst are F32, the matrix F32 or BF16 (got x %s, w %s, dst %s)", what, dtype_name(x->dtype),
                     dtype_name(w->dtype), dtype_name(dst->dtype));
  if (dst == x || dst == w || dst == alpha) return set_error(UGHIP_ERR_INVALID, "%s: dst aliases an operand", what);
  if (m > 0x7fffffffull || rows > 0x7fffffffull || k > 0x7fffffffull / 3) return set_error(UGHIP_ERR_INVALID, "%s: shape too large", what);
  const size_t out_cols = kind == GemmEpilogue::SWIGLU ? rows / 2 : rows;
  if (x->len < m * k || w->len < rows * k || dst->len < m * out_cols || (residual && residual->len < m * rows) || (alpha && alpha->len < k))
    return set_error(UGHIP_ERR_BOUNDS, "%s: a buffer is too short for m %zu, n %zu, k %zu", what, m, out_cols, k);
  RowsAround ar;
  if (alpha) {
    if (int rc = device_activate(dev)) return rc;
    if (int rc = grow_rows_ws(dev, m * k * sizeof(float))) return rc;
    ar.alpha = static_cast<const float*>(alpha->ptr), ar.eps = eps, ar.xn = static_cast<float*>(dev->rows_ws);
  }
  return linear_rows_core(dev, what, static_cast<const float*>(x->ptr), w, residual ? static_cast<const float*>(residual->ptr) : nullptr, static_cast<float*>(dst->ptr), m,
                          rows, k, kind, product, &ar);
}

// dst[m, n] = silu(y gate^T) * (y up^T) w_down^T + residual with y = x, or RMSNorm(x) when alpha is given: the two products of
// an MLP block (model.rs:160-168 between the residual adds of 366-372) with what lies between them kept in the device's own
// scratch -- as the three bf16 planes the second product reads where both run on planes, else as f32 rows.
static int mlp_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps, const ughip_slice* w_gate_up, const ughip_slice* w_down,
                    const ughip_slice* residual, ughip_slice* dst, size_t m, size_t n, size_t inter, size_t k, int product) {
  const char* what = "rms_mlp_rows";
  if (!dev || !x || !w_gate_up || !w_down || !residual || !dst) return set_error(UGHIP_ERR_INVALID, "%s: null argument", what);
  if (x->dtype != UGHIP_F32 || dst->dtype != UGHIP_F32 || residual->dtype != UGHIP_F32 || (alpha && alpha->dtype != UGHIP_F32) ||
      (w_gate_up->dtype != UGHIP_F32 && w_gate_up->dtype != UGHIP_BF16) || w_down->dtype != w_gate_up->dtype)
    return set_error(UGHIP_ERR_INVALID, "%s: x, alpha, residual and dst are F32, the two matrices both F32 or both BF16", what);
  if (dst == x || dst == alpha || dst == w_gate_up || dst == w_down) return set_error(UGHIP_ERR_INVALID, "%s: dst aliases an operand", what);
  if (m > 0x7fffffffull || n > 0x7fffffffull || inter > 0x7fffffffull / 3 || k > 0x7fffffffull / 3) return set_error(UGHIP_ERR_INVALID, "%s: shape too large", what);
  if (x->len < m * k || w_gate_up->len < 2 * inter * k || w_down->len < n * inter || dst->len < m * n || residual->len < m * n || (alpha && alpha->len < k))
    return set_error(UGHIP_ERR_BOUNDS, "%s: a buffer is too short for m %zu, n %zu, inter %zu, k %zu", what, m, n, inter, k);
  if (m == 0 || n == 0) return UGHIP_OK;
  if (inter == 0 || inter % 8 != 0) return set_error(UGHIP_ERR_UNSUPPORTED, "%s: inter %% 8 == 0 (got %zu)", what, inter);
  // scratch: [normalised rows, f32, if any | what the first product leaves: m * inter elements as f32 (4 bytes) or as planes (6)]
  const size_t xn_bytes = alpha ? (m * k * sizeof(float) + 255) & ~(size_t)255 : 0;
  if (int rc = device_activate(dev)) return rc;
  if (int rc = grow_rows_ws(dev, xn_bytes + m * inter * 6)) return rc;
  float* h = reinterpret_cast<float*>(static_cast<char*>(dev->rows_ws) + xn_bytes);
  RowsAround first, second;
  if (alpha) first.alpha = static_cast<const float*>(alpha->ptr), first.eps = eps, first.xn = static_cast<float*>(dev->rows_ws);
  const bool x3 = product == UGHIP_PRODUCT_BF16X3;
  if (x3 && w_down->dtype == UGHIP_BF16 && inter % 64 == 0 && n % 8 == 0 && m >= 2) {
    // the second product reads planes unless it is one that splits its rows itself
    const MMArgs pd = rows_args(h, w_down->ptr, dst->ptr, m, n, inter, true);
    if (gemm_tiled_supported(UGHIP_BF16, pd, 1, false) &&
        rows_route(pd, UGHIP_BF16, true, GemmEpilogue::ADD, h, w_down->ptr, dst->ptr, residual->ptr, m, n, inter, dev->num_cus).kind != RowsRoute::X3_ROWS)
      first.planes_out = reinterpret_cast<uint16_t*>(h);
  }
  if (int rc = linear_rows_core(dev, what, static_cast<const float*>(x->ptr), w_gate_up, nullptr, h, m, 2 * inter, k, GemmEpilogue::SWIGLU, product, &first)) return rc;
  char first_kernel[160];
  snprintf(first_kernel, sizeof first_kernel, "%s", ughip_last_kernel());
  if (first.wrote_planes) second.planes_in = reinterpret_cast<const uint16_t*>(h);
  if (int rc = linear_rows_core(dev, what, h, w_down, static_cast<const float*>(residual->ptr), static_cast<float*>(dst->ptr), m, n, inter, GemmEpilogue::ADD, product, &second))
    return rc;
  char second_kernel[160];
  snprintf(second_kernel, sizeof second_kernel, "%s", ughip_last_kernel());
  note_kernel("%s -> %s", first_kernel, second_kernel);
  return UGHIP_OK;
}

// The kernel ughip_matmul would launch for contiguous operands of these shapes (rhs_nk: the rhs stored [n, k], i.e. strides (1, k)),
// by the name ughip_last_kernel() reports after the launch.  Needs no device: the choice depends on shapes and on the cost models.
extern "C" int ughip_matmul_plan(int dtype, int rhs_dtype, size_t b, size_t m, size_t n, size_t k, int rhs_nk, char* buf, size_t buf_len) {
  if (!buf || !buf_len) return set_error(UGHIP_ERR_INVALID, "matmul_plan: no buffer");
  const bool mixed = dtype == UGHIP_F32 && rhs_dtype == UGHIP_BF16;
  if ((!mixed && dtype != rhs_dtype) || (dtype != UGHIP_F32 && dtype != UGHIP_BF16 && dtype != UGHIP_F16))
    return set_error(UGHIP_ERR_UNSUPPORTED, "matmul_plan: dtypes %s x %s", dtype_name(dtype), dtype_name(rhs_dtype));
  if (!b || !m || !n || !k || b > 65535 || m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "matmul_plan: bad shape");
  MMArgs p;
  p.M = (int)m, p.N = (int)n, p.K = (int)k;
  p.a_rs = (long long)k, p.a_cs = 1;
  p.b_rs = rhs_nk ? 1 : (long long)n, p.b_cs = rhs_nk ? (long long)k : 1;
  p.a_bs = (long long)(m * k), p.b_bs = (long long)(n * k), p.c_bs = (long long)(m * n);
  p.a = p.b = reinterpret_cast<const void*>(uintptr_t(1) << 20);  // stand-ins with the alignment every allocation has; never dereferenced
  p.c = reinterpret_cast<void*>(uintptr_t(1) << 20);
  int tile = 0;
  const char* tn = dtype == UGHIP_F32 ? "f32" : dtype == UGHIP_F16 ? "f16" : "bf16";
  switch (matmul_route(dtype, mixed, p, b, 0, 0, &tile)) {
    case ROUTE_UNSUPPORTED: return set_error(UGHIP_ERR_UNSUPPORTED, "matmul_plan: an F32 product with a BF16 rhs needs an [n, k]-major rhs and k %% 32 == 0");
    case ROUTE_GEMV_NT: snprintf(buf, buf_len, "gemv_nt<%s>", tn); break;
    case ROUTE_GEMV_NN: snprintf(buf, buf_len, "gemv_nn<f32>"); break;
    case ROUTE_DMA: gemm_dma_name(dtype, p, tile, buf, buf_len); break;
    case ROUTE_DMA_F32: gemm_dma_f32_name(p, buf, buf_len); break;
    case ROUTE_X6: {
      MMArgs q;
      matmul_x6_plan(p, b, 0, 0, &q);
      gemm_dma_planes6_name(q, tile, buf, buf_len);
      break;
    }
    case ROUTE_TILED: gemm_tiled_name(dtype, p, b, mixed, nullptr, buf, buf_len); break;
    default: snprintf(buf, buf_len, "gemm_any<%s>", tn); break;
  }
  return UGHIP_OK;
}

// The kernel ughip_linear_rows (form 0), ughip_linear_add_rows (1) or ughip_linear_swiglu_rows (2; n output columns from 2 n matrix
// rows) would launch for m rows, by the name ughip_last_kernel() reports after the launch.  Needs no device (256 CUs assumed).
extern "C" int ughip_linear_rows_plan(int w_dtype, int product, int form, size_t m, size_t n, size_t k, char* buf, size_t buf_len) {
  if (!buf || !buf_len) return set_error(UGHIP_ERR_INVALID, "linear_rows_plan: no buffer");
  if ((w_dtype != UGHIP_F32 && w_dtype != UGHIP_BF16) || (product != UGHIP_PRODUCT_F32 && product != UGHIP_PRODUCT_BF16X3) || form < 0 || form > 2 ||
      (product == UGHIP_PRODUCT_BF16X3 && w_dtype != UGHIP_BF16))
    return set_error(UGHIP_ERR_INVALID, "linear_rows_plan: bad dtype, product or form");
  const size_t rows = form == 2 ? 2 * n : n;
  if (!m || !n || !k || m > 0x7fffffffull || rows > 0x7fffffffull || k > 0x7fffffffull / 3) return set_error(UGHIP_ERR_INVALID, "linear_rows_plan: bad shape");
  const GemmEpilogue::Kind kind = form == 2 ? GemmEpilogue::SWIGLU : form == 1 ? GemmEpilogue::ADD : GemmEpilogue::NONE;
  const bool x3 = product == UGHIP_PRODUCT_BF16X3, mixed = !x3 && w_dtype == UGHIP_BF16;
  const int dtype = x3 ? UGHIP_BF16 : UGHIP_F32;
  void* stand_in = reinterpret_cast<void*>(uintptr_t(1) << 20);  // the alignment every allocation has; never dereferenced
  MMArgs p;
  p.M = (int)m, p.N = (int)rows, p.K = (int)(x3 ? 3 * k : k);
  p.a_rs = (long long)(x3 ? 3 * k : k), p.a_cs = 1, p.b_rs = 1, p.b_cs = (long long)k;
  p.a_bs = (long long)(m * (x3 ? 3 * k : k)), p.b_bs = (long long)(rows * k), p.c_bs = (long long)(m * rows);
  p.a = p.b = stand_in, p.c = stand_in;
  if (x3) p.b_k_div = 3;
  const size_t min_rows = w_dtype == UGHIP_BF16 ? 2 : 9;
  if (m < min_rows || rows % 8 != 0 || (kind == GemmEpilogue::SWIGLU && rows % 16 != 0) || (x3 && k % 64 != 0) || !gemm_tiled_supported(dtype, p, 1, mixed))
    return set_error(UGHIP_ERR_UNSUPPORTED, "linear_rows_plan: a shape the entry points refuse (m %zu, n %zu, k %zu)", m, n, k);
  GemmEpilogue epi{kind, form == 1 ? static_cast<const float*>(stand_in) : nullptr};
  epi.out_f32 = x3;
  const RowsRoute route = rows_route(p, dtype, x3, kind, stand_in, stand_in, stand_in, form == 1 ? stand_in : nullptr, m, rows, k, 256);
  if (route.kind == RowsRoute::X3_ROWS) {
    rows_x3_name(route.x3, kind, buf, buf_len);
  } else if (route.kind == RowsRoute::DMA_PLANES) {
    const bool fold = route.dma_split > 1 || kind == GemmEpilogue::SWIGLU;
    int bm = 256, bn = route.dma_tile == 256 ? 256 : 128;
    if (route.dma_tile == 64) bm = 128;
    char split[24] = "";
    if (route.dma_split > 1) snprintf(split, sizeof split, ",splitK=%d", route.dma_split);
    snprintf(buf, buf_len, "gemm_dma4<bf16,NT,%dx%d,256t,3 planes%s,f32 out%s>", bm, bn, split, dma_planes_tail(kind, fold, form == 1));
  } else {
    gemm_tiled_name(dtype, p, 1, mixed, &epi, buf, buf_len);
  }
  return UGHIP_OK;
}

extern "C" int ughip_linear_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* w, ughip_slice* dst, size_t m, size_t n, size_t k, int product) {
  return linear_rows(dev, "linear_rows", x, w, nullptr, dst, m, n, k, GemmEpilogue::NONE, product);
}

extern "C" int ughip_linear_add_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* w, const ughip_slice* residual, ughip_slice* dst, size_t m,
                                     size_t n, size_t k, int product) {
  return linear_rows(dev, "linear_add_rows", x, w, residual, dst, m, n, k, GemmEpilogue::ADD, product);
}

extern "C" int ughip_linear_swiglu_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* w, ughip_slice* dst, size_t m, size_t n, size_t k,
                                        int product) {
  if (n > 0x3fffffffull) return set_error(UGHIP_ERR_INVALID, "linear_swiglu_rows: shape too large");
  return linear_rows(dev, "linear_swiglu_rows", x, w, nullptr, dst, m, 2 * n, k, GemmEpilogue::SWIGLU, product);
}

extern "C" int ughip_rms_linear_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps, const ughip_slice* w, ughip_slice* dst, size_t m,
                                     size_t n, size_t k, int product) {
  if (!alpha) return set_error(UGHIP_ERR_INVALID, "rms_linear_rows: null argument");
  return linear_rows(dev, "rms_linear_rows", x, w, nullptr, dst, m, n, k, GemmEpilogue::NONE, product, alpha, eps);
}

extern "C" int ughip_rms_mlp_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps, const ughip_slice* w_gate_up, const ughip_slice* w_down,
                                  const ughip_slice* residual, ughip_slice* dst, size_t m, size_t n, size_t inter, size_t k, int product) {
  return mlp_rows(dev, x, alpha, eps, w_gate_up, w_down, residual, dst, m, n, inter, k, product);
}

namespace ughip {

int rows_scratch(ughip_device* dev, size_t bytes, void** out) {
  if (int rc = grow_rows_ws(dev, bytes)) return rc;
  *out = dev->rows_ws;
  return UGHIP_OK;
}

bool rows_add_product_reads_planes(ughip_device* dev, const ughip_slice* w, const void* x, const void* residual, const void* dst, size_t m, size_t n, size_t k, int product) {
  if (product != UGHIP_PRODUCT_BF16X3 || !w || w->dtype != UGHIP_BF16 || k % 64 != 0 || n % 8 != 0 || m < 2 || m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull / 3)
    return false;
  const MMArgs p = rows_args(x, w->ptr, const_cast<void*>(dst), m, n, k, true);
  return gemm_tiled_supported(UGHIP_BF16, p, 1, false) &&
         rows_route(p, UGHIP_BF16, true, GemmEpilogue::ADD, x, w->ptr, dst, residual, m, n, k, dev->num_cus).kind != RowsRoute::X3_ROWS;
}

int rows_add_product_from(ughip_device* dev, const char* what, const float* x, const uint16_t* planes, const ughip_slice* w, const float* residual, float* dst, size_t m,
                          size_t n, size_t k, int product) {
  RowsAround ar;
  ar.planes_in = planes;
  return linear_rows_core(dev, what, x, w, residual, dst, m, n, k, GemmEpilogue::ADD, product, &ar);
}

}  // namespace ughip
