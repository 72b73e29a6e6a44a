// Row-vector projections of a decode step with their neighbours folded in (f32, one input row):
//
//   ughip_gemv_multi    y = [x W_0^T | x W_1^T | x W_2^T]: up to three matrices over the same x in one
//                       launch, results side by side (the q / k / v projections of
//                       ug-llama/src/model.rs:206-208)
//   ughip_gemv_gate_up  y = silu(x G^T) * (x U^T), silu(g) = g / (1 + exp(-g))
//                       (model.rs:160-168 up to the down projection, written as in model.rs:99-109)
//   ughip_gemv_add      y = x W^T + r   (o_proj / down_proj followed by the residual add, model.rs:366-372)
//   ughip_rms_gemv_multi, ughip_rms_gemv_gate_up: the first two with RMSNorm (model.rs:32-50) applied to x
//                       on the way in (the norms in front of attention, the MLP and the output head)
//
// One token's projections are 6-46 MB matrix streams behind 2-3 us launches; these entry points
// remove launches and the small vectors that would travel between them, nothing else: every
// product is the same fixed-order f32 sum a separate ughip_matmul computes, the epilogues are
// the same f32 operations the lazy graph would run on the rounded products.
//
// The matrices may be stored as BF16 (all of one call alike) while x, the sums and y stay F32: a
// bf16 widens to f32 exactly, so the result is the one the F32 kernel gives on the same values (bit
// for bit where both run the same kernel, to the rounding of another order of the sums where the
// BF16 rows have a kernel of their own, below), from half the bytes - decode streams every weight
// once per token and nothing else of that size.  (ug's Device::matmul wants one dtype for all three operands, ug-core/src/lib.rs:62-70;
// a checkpoint stored in bf16 is widened at load time, ug-core/src/safetensors.rs:120-271.)
//
// F32 matrices (and BF16 rows the kernel below does not take): KS waves share one output column, each
// walking every KS-th 64-lane slab of k with four 128-bit loads in flight per lane and matrix; a
// workgroup of 4 waves covers 4 / KS columns.  BF16 matrices with rows of 512 .. 8192 elements:
// fused_gemv_bf16_rows, x in registers and R rows per workgroup (described where it is defined).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdlib>

#include "internal.h"
#include "ughip.h"
#include "wave_ops.h"

using namespace ughip;

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

enum { MODE_MULTI = 0, MODE_GATE_UP = 1, MODE_ADD = 2 };

struct FusedArgs {
  const float* x;
  const void* w[3];  // [n_i, k] row-major, float or bf16 (the kernel's WT)
  float* y[3];
  int col_end[3];  // MODE_MULTI: matrix i owns the columns col_end[i-1] .. col_end[i] - 1 of the grid
  int n_cols;      // columns of the grid
  int k;
  const float* residual;
  const float* alpha;  // RMS variants: y uses x / sqrt(mean(x^2) + eps) * alpha in place of x
  float eps;
};

// Four consecutive matrix elements as f32.  Every matrix element is read once per launch: the loads do not
// claim cache lines (the 262 MB head: 42.1 -> 38.6 us).
template <typename WT>
__device__ __forceinline__ f32x4 load_w4(const WT* p);
template <>
__device__ __forceinline__ f32x4 load_w4<float>(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
}
template <>
__device__ __forceinline__ f32x4 load_w4<uint16_t>(const uint16_t* p) {
  const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
  return f32x4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u)};
}

__device__ __forceinline__ float dot4(const f32x4& w, const f32x4& x, float acc) {
  acc += w.x * x.x;
  acc += w.y * x.y;
  acc += w.z * x.z;
  acc += w.w * x.w;
  return acc;
}

template <typename WT, int KS, int MODE>
__global__ void __launch_bounds__(256) fused_gemv(FusedArgs a) {
  __shared__ float part[4][2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * (4 / KS) + wave / KS, ks = wave % KS;
  const bool live = col < a.n_cols;
  // which matrix and which of its rows this column is
  const WT* __restrict__ W0 = nullptr;
  const WT* __restrict__ W1 = nullptr;
  float* __restrict__ Y = nullptr;
  if (live) {
    int m = 0, first = 0;
    if (MODE == MODE_MULTI) {
      if (col >= a.col_end[0]) m = 1, first = a.col_end[0];
      if (col >= a.col_end[1]) m = 2, first = a.col_end[1];
    }
    const int row = col - first;
    W0 = static_cast<const WT*>(a.w[m]) + (size_t)row * a.k;
    if (MODE == MODE_GATE_UP) W1 = static_cast<const WT*>(a.w[1]) + (size_t)row * a.k;
    Y = a.y[m] + row;
  }
  float acc0 = 0.f, acc1 = 0.f;
  if (live) {
    const float* __restrict__ X = a.x;
    constexpr int stride = 64 * 4 * KS;
    int k = (ks * 64 + lane) * 4;
    // four slabs per trip, all requested before the first is used; slabs past the end of the row
    // are skipped lane by lane (a short row must not turn into a chain of single loads)
    for (; k < a.k; k += 4 * stride) {
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
      f32x4 w[4], u[4], x[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ki = k + i * stride;
        w[i] = u[i] = x[i] = zero;
        if (ki < a.k) {
          w[i] = load_w4<WT>(W0 + ki);
          if (MODE == MODE_GATE_UP) u[i] = load_w4<WT>(W1 + ki);
          x[i] = *reinterpret_cast<const f32x4*>(X + ki);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) acc0 = dot4(w[i], x[i], acc0);
      if (MODE == MODE_GATE_UP) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc1 = dot4(u[i], x[i], acc1);
      }
    }
  }
  acc0 = wave_sum(acc0);
  if (MODE == MODE_GATE_UP) acc1 = wave_sum(acc1);
  if (KS > 1) {
    if (lane == 0) {
      part[wave][0] = acc0;
      part[wave][1] = acc1;
    }
    __syncthreads();
    if (ks != 0) return;
    acc0 = part[wave][0];
    acc1 = part[wave][1];
#pragma unroll
    for (int j = 1; j < KS; ++j) {
      acc0 += part[wave + j][0];
      acc1 += part[wave + j][1];
    }
  }
  if (!live || lane != 0) return;
  if (MODE == MODE_GATE_UP) *Y = acc0 / (1.f + expf(-acc0)) * acc1;
  else if (MODE == MODE_ADD) *Y = acc0 + a.residual[col];
  else *Y = acc0;
}

// The same with RMSNorm (ug-llama/src/model.rs:32-50: x / sqrt(mean(x^2) + eps) * alpha) applied to x
// first.  The row is short (k <= 256 * RMS_SLABS floats): a wave requests all of its matrix loads,
// the workgroup normalises the row once into LDS in their shadow, then every wave multiplies.
constexpr int RMS_SLABS = 16;

// FULL: the row has exactly 256 * SLABS elements, no slab needs a bounds check (the guards and
// the zero fills behind them are most of the instructions of the general form, and at 4 cycles per
// wave instruction these kernels are not far from being bound by them).
template <typename WT, int KS, int MODE, int SLABS, bool FULL>
__global__ void __launch_bounds__(256) fused_rms_gemv(FusedArgs a) {
  constexpr int NVW = SLABS / KS;  // slabs of 256 floats per wave
  const int klen = FULL ? SLABS * 256 : a.k;
  __shared__ float part[4][2];
  __shared__ float ssum[4];
  __shared__ f32x4 xs[SLABS * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * (4 / KS) + wave / KS, ks = wave % KS;
  const bool live = col < a.n_cols;
  // Loads come back in the order they were issued.  The row and the norm weights (cache hits, thread t
  // owns elements 4 t .. 4 t + 3 of every 1024) are requested first so that the norm below runs while
  // the matrix rows, the long pole, are still on their way from memory.
  const float* __restrict__ X = a.x;
  constexpr int PER_T = SLABS / 4;
  f32x4 xl[PER_T], al[PER_T];
#pragma unroll
  for (int i = 0; i < PER_T; ++i) {
    const int k = (i * 256 + (int)threadIdx.x) * 4;
    xl[i] = al[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (FULL || k < klen) {
      xl[i] = *reinterpret_cast<const f32x4*>(X + k);
      al[i] = *reinterpret_cast<const f32x4*>(a.alpha + k);
    }
  }
  float* __restrict__ Y = nullptr;
  f32x4 w0[NVW], w1[NVW];
#pragma unroll
  for (int j = 0; j < NVW; ++j) w0[j] = w1[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (live) {
    int mtx = 0, first = 0;
    if (MODE == MODE_MULTI) {
      if (col >= a.col_end[0]) mtx = 1, first = a.col_end[0];
      if (col >= a.col_end[1]) mtx = 2, first = a.col_end[1];
    }
    const int row = col - first;
    const WT* __restrict__ W0 = static_cast<const WT*>(a.w[mtx]) + (size_t)row * klen;
    const WT* __restrict__ W1 = MODE == MODE_GATE_UP ? static_cast<const WT*>(a.w[1]) + (size_t)row * klen : nullptr;
    Y = a.y[mtx] + row;
#pragma unroll
    for (int j = 0; j < NVW; ++j) {
      const int k = ((j * KS + ks) * 64 + lane) * 4;
      if (FULL || k < klen) {
        w0[j] = load_w4<WT>(W0 + k);
        if (MODE == MODE_GATE_UP) w1[j] = load_w4<WT>(W1 + k);
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // the workgroup normalises the row once, into LDS
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PER_T; ++i) {
    ss += xl[i].x * xl[i].x;
    ss += xl[i].y * xl[i].y;
    ss += xl[i].z * xl[i].z;
    ss += xl[i].w * xl[i].w;
  }
  ss = wave_sum(ss);
  if (lane == 0) ssum[wave] = ss;
  __syncthreads();
  ss = (ssum[0] + ssum[1]) + (ssum[2] + ssum[3]);
  const float inv = 1.f / sqrtf(ss * (1.f / (float)klen) + a.eps);  // one division per thread; x / m as x * (1 / m) is within an ulp
#pragma unroll
  for (int i = 0; i < PER_T; ++i) {
    const int k = (i * 256 + (int)threadIdx.x) * 4;
    if (FULL || k < klen) xs[i * 256 + threadIdx.x] = f32x4{xl[i].x * inv * al[i].x, xl[i].y * inv * al[i].y, xl[i].z * inv * al[i].z, xl[i].w * inv * al[i].w};
  }
  __syncthreads();
  float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
  for (int j = 0; j < NVW; ++j) {
    const int k4 = (j * KS + ks) * 64 + lane;
    if (FULL || k4 * 4 < klen) {
      const f32x4 xn = xs[k4];
      acc0 = dot4(w0[j], xn, acc0);
      if (MODE == MODE_GATE_UP) acc1 = dot4(w1[j], xn, acc1);
    }
  }
  acc0 = wave_sum(acc0);
  if (MODE == MODE_GATE_UP) acc1 = wave_sum(acc1);
  if (KS > 1) {
    if (lane == 0) {
      part[wave][0] = acc0;
      part[wave][1] = acc1;
    }
    __syncthreads();
    if (ks != 0) return;
    acc0 = part[wave][0];
    acc1 = part[wave][1];
#pragma unroll
    for (int j = 1; j < KS; ++j) {
      acc0 += part[wave + j][0];
      acc1 += part[wave + j][1];
    }
  }
  if (!live || lane != 0) return;
  if (MODE == MODE_GATE_UP) *Y = acc0 / (1.f + expf(-acc0)) * acc1;
  else *Y = acc0;
}

// BF16 matrices, rows of 512 .. 8192 elements (a multiple of 8): thread t of the workgroup keeps x[8 t .. 8 t + 7] of
// every 2048 elements in registers and the workgroup walks R matrix rows with one 128-bit load per thread, row and
// 2048 elements.  Against the kernels above (64-bit loads, x fetched again with every slab) the matrix streams
// 10-30 % faster at the decode shapes: half the load instructions per byte and no traffic for x beside the matrix.
// The sums run in another order than the F32 kernels' (eight consecutive elements per lane), so a BF16 matrix no
// longer gives the bits of the F32 matrix holding the same values: both stay within the k * eps bound of the exact product.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float dot8_bf16(const u32x4& v, const f32x4& xa, const f32x4& xb, float acc) {
  acc += __uint_as_float(v.x << 16) * xa.x;
  acc += __uint_as_float(v.x & 0xffff0000u) * xa.y;
  acc += __uint_as_float(v.y << 16) * xa.z;
  acc += __uint_as_float(v.y & 0xffff0000u) * xa.w;
  acc += __uint_as_float(v.z << 16) * xb.x;
  acc += __uint_as_float(v.z & 0xffff0000u) * xb.y;
  acc += __uint_as_float(v.w << 16) * xb.z;
  acc += __uint_as_float(v.w & 0xffff0000u) * xb.w;
  return acc;
}

constexpr int ROWS_KT_MAX = 4;  // rows of up to 4 * 2048 elements

template <int R, int KT, int MODE, bool RMS>
__global__ void __launch_bounds__(256) fused_gemv_bf16_rows(FusedArgs a) {
  constexpr int NM = MODE == MODE_GATE_UP ? 2 : 1;
  __shared__ float part[4][NM * R];
  __shared__ float ssum[4];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int klen = a.k;
  const int col0 = blockIdx.x * R;
  // Loads come back in the order they were issued: x (and the norm weights), cache hits, go first so that the
  // norm runs while the matrix rows are on their way.
  f32x4 xa[KT], xb[KT], ala[KT], alb[KT];
#pragma unroll
  for (int c = 0; c < KT; ++c) {
    const int kk = c * 2048 + t * 8;
    xa[c] = xb[c] = ala[c] = alb[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (kk < klen) {
      xa[c] = *reinterpret_cast<const f32x4*>(a.x + kk);
      xb[c] = *reinterpret_cast<const f32x4*>(a.x + kk + 4);
      if (RMS) {
        ala[c] = *reinterpret_cast<const f32x4*>(a.alpha + kk);
        alb[c] = *reinterpret_cast<const f32x4*>(a.alpha + kk + 4);
      }
    }
  }
  u32x4 w[NM][R][KT];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int col = col0 + r;
    int mtx = 0, first = 0;
    if (MODE == MODE_MULTI) {
      if (col >= a.col_end[0]) mtx = 1, first = a.col_end[0];
      if (col >= a.col_end[1]) mtx = 2, first = a.col_end[1];
    }
    const bool live = col < a.n_cols;
    const size_t at = live ? (size_t)(col - first) * klen : 0;
    const uint16_t* __restrict__ W0 = static_cast<const uint16_t*>(a.w[live ? mtx : 0]) + at;
    const uint16_t* __restrict__ W1 = MODE == MODE_GATE_UP ? static_cast<const uint16_t*>(a.w[1]) + at : nullptr;
#pragma unroll
    for (int c = 0; c < KT; ++c) {
      const int kk = c * 2048 + t * 8;
      const bool ok = live && kk < klen;
      w[0][r][c] = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(W0 + kk)) : u32x4{0, 0, 0, 0};
      if (MODE == MODE_GATE_UP) w[1][r][c] = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(W1 + kk)) : u32x4{0, 0, 0, 0};
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  if (RMS) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < KT; ++c) {
      ss += xa[c].x * xa[c].x;
      ss += xa[c].y * xa[c].y;
      ss += xa[c].z * xa[c].z;
      ss += xa[c].w * xa[c].w;
      ss += xb[c].x * xb[c].x;
      ss += xb[c].y * xb[c].y;
      ss += xb[c].z * xb[c].z;
      ss += xb[c].w * xb[c].w;
    }
    ss = wave_sum(ss);
    if (lane == 0) ssum[wave] = ss;
    __syncthreads();
    ss = (ssum[0] + ssum[1]) + (ssum[2] + ssum[3]);
    const float inv = 1.f / sqrtf(ss * (1.f / (float)klen) + a.eps);
#pragma unroll
    for (int c = 0; c < KT; ++c) {
      xa[c] = f32x4{xa[c].x * inv * ala[c].x, xa[c].y * inv * ala[c].y, xa[c].z * inv * ala[c].z, xa[c].w * inv * ala[c].w};
      xb[c] = f32x4{xb[c].x * inv * alb[c].x, xb[c].y * inv * alb[c].y, xb[c].z * inv * alb[c].z, xb[c].w * inv * alb[c].w};
    }
  }
  float acc[NM][R];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < KT; ++c) s = dot8_bf16(w[m][r][c], xa[c], xb[c], s);
      acc[m][r] = wave_sum(s);
    }
  if (lane == 0) {
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) part[wave][m * R + r] = acc[m][r];
  }
  __syncthreads();
  const int col = col0 + t;
  if (t >= R || col >= a.n_cols) return;
  const float s0 = (part[0][t] + part[1][t]) + (part[2][t] + part[3][t]);
  if (MODE == MODE_GATE_UP) {
    const float s1 = (part[0][R + t] + part[1][R + t]) + (part[2][R + t] + part[3][R + t]);
    a.y[0][col] = s0 / (1.f + expf(-s0)) * s1;
  } else if (MODE == MODE_ADD) {
    a.y[0][col] = s0 + a.residual[col];
  } else {
    int mtx = 0, first = 0;
    if (col >= a.col_end[0]) mtx = 1, first = a.col_end[0];
    if (col >= a.col_end[1]) mtx = 2, first = a.col_end[1];
    a.y[mtx][col - first] = s0;
  }
}

template <int R, int KT, int MODE, bool RMS>
void launch_bf16_rows_r(hipStream_t st, const FusedArgs& a) {
  constexpr int NM = MODE == MODE_GATE_UP ? 2 : 1;
  if constexpr (R * KT * NM <= 16) {  // 64 registers of matrix elements per thread at most
    const unsigned grid = ((unsigned)a.n_cols + R - 1) / R;
    fused_gemv_bf16_rows<R, KT, MODE, RMS><<<grid, 256, 0, st>>>(a);
  } else {
    launch_bf16_rows_r<R / 2, KT, MODE, RMS>(st, a);
  }
}

template <int MODE, bool RMS, int KT>
void launch_bf16_rows_kt(hipStream_t st, const FusedArgs& a) {
  // Rows per workgroup: every workgroup fetches x (and normalises it) once for its rows, so more rows mean less traffic
  // beside the matrix; fewer rows mean more workgroups to spread a small matrix over the chip.
  constexpr int NM = MODE == MODE_GATE_UP ? 2 : 1;
  // Measured at the decode shapes (2048 .. 32000 rows of 2048 and 5632 elements): 2 rows, 4 where a row takes several
  // loads per thread, 8 for a matrix of very many short rows (the output head).
  int r = 2;
  if (NM == 1 && KT >= 2) r = 4;
  if (a.n_cols >= 16384) r = NM == 1 && KT == 1 ? 8 : 4;
  if (long long v; tune_get(TUNE_GEMV_ROWS, &v)) r = (int)v;  // tuning aid: 1, 2, 4 or 8
  if (r >= 8) launch_bf16_rows_r<8, KT, MODE, RMS>(st, a);
  else if (r >= 4) launch_bf16_rows_r<4, KT, MODE, RMS>(st, a);
  else if (r >= 2) launch_bf16_rows_r<2, KT, MODE, RMS>(st, a);
  else launch_bf16_rows_r<1, KT, MODE, RMS>(st, a);
}

template <int MODE, bool RMS>
void launch_bf16_rows(hipStream_t st, const FusedArgs& a) {
  const int kt = (a.k + 2047) / 2048;
  if (kt == 1) launch_bf16_rows_kt<MODE, RMS, 1>(st, a);
  else if (kt == 2) launch_bf16_rows_kt<MODE, RMS, 2>(st, a);
  else if (kt == 3) launch_bf16_rows_kt<MODE, RMS, 3>(st, a);
  else launch_bf16_rows_kt<MODE, RMS, 4>(st, a);
}

bool bf16_rows_fit(const FusedArgs& a) {
  if (long long v; tune_get(TUNE_GEMV_BF16_ROWS, &v) && v == 0) return false;  // tuning aid: the older kernels
  return a.k % 8 == 0 && a.k >= 512 && a.k <= 2048 * ROWS_KT_MAX;
}

int pick_ks(size_t cols, size_t k) {
  // enough waves to hide HBM latency: about 8192 over the chip
  int ks = cols <= 2048 ? 4 : cols <= 6144 ? 2 : 1;
  if (long long v; tune_get(TUNE_GEMV_KS, &v)) ks = (int)v;  // tuning aid: 1, 2 or 4
  if (ks != 1 && ks != 2 && ks != 4) ks = 1;
  while (ks > 1 && k < (size_t)64 * 4 * ks) ks >>= 1;
  return ks;
}

template <typename WT, int MODE>
void launch_t(hipStream_t st, const FusedArgs& a) {
  const int ks = pick_ks((size_t)a.n_cols, (size_t)a.k);  // measured: gate/up (two rows per wave) also does best with the plain rule
  const unsigned per_wg = 4 / ks;
  const unsigned grid = ((unsigned)a.n_cols + per_wg - 1) / per_wg;
  if (a.alpha) {
    if (MODE == MODE_ADD) return;  // not built (the residual projections read attention / SwiGLU outputs, not a norm)
    constexpr int M = MODE == MODE_ADD ? MODE_MULTI : MODE;
    const bool small = a.k <= 256 * 8, full = a.k == 256 * 8 || a.k == 256 * 16;
#define UGHIP_RMS_GO(KS_)                                                                             \
  do {                                                                                                \
    if (small && full) fused_rms_gemv<WT, KS_, M, 8, true><<<grid, 256, 0, st>>>(a);                  \
    else if (small) fused_rms_gemv<WT, KS_, M, 8, false><<<grid, 256, 0, st>>>(a);                    \
    else if (full) fused_rms_gemv<WT, KS_, M, 16, true><<<grid, 256, 0, st>>>(a);                     \
    else fused_rms_gemv<WT, KS_, M, 16, false><<<grid, 256, 0, st>>>(a);                              \
  } while (0)
    if (ks == 4) UGHIP_RMS_GO(4);
    else if (ks == 2) UGHIP_RMS_GO(2);
    else UGHIP_RMS_GO(1);
#undef UGHIP_RMS_GO
    return;
  }
  if (ks == 4) fused_gemv<WT, 4, MODE><<<grid, 256, 0, st>>>(a);
  else if (ks == 2) fused_gemv<WT, 2, MODE><<<grid, 256, 0, st>>>(a);
  else fused_gemv<WT, 1, MODE><<<grid, 256, 0, st>>>(a);
}

template <int MODE>
hipError_t launch(hipStream_t st, const FusedArgs& a, int w_dtype) {
  // a norm in front of the residual form: no entry point asks for it and no kernel is built for it -- an error, not a launch
  // that silently does nothing
  if (MODE == MODE_ADD && a.alpha) return hipErrorInvalidValue;
  if (w_dtype == UGHIP_BF16 && bf16_rows_fit(a)) {
    if (a.alpha) {
      constexpr int M = MODE == MODE_ADD ? MODE_MULTI : MODE;
      launch_bf16_rows<M, true>(st, a);
    } else {
      launch_bf16_rows<MODE, false>(st, a);
    }
    return hipGetLastError();
  }
  if (w_dtype == UGHIP_BF16) launch_t<uint16_t, MODE>(st, a);
  else launch_t<float, MODE>(st, a);
  return hipGetLastError();
}

int check(const ughip_device* dev, const ughip_slice* s, size_t need, const char* what) {
  if (!s) return set_error(UGHIP_ERR_INVALID, "%s: null slice", what);
  if (s->dev != dev) return set_error(UGHIP_ERR_INVALID, "%s: slice lives on another device", what);
  if (s->dtype != UGHIP_F32) return set_error(UGHIP_ERR_UNSUPPORTED, "%s: dtype %s, this entry point is built for F32", what, dtype_name(s->dtype));
  if (s->len < need) return set_error(UGHIP_ERR_BOUNDS, "%s: slice has %zu elements, op needs %zu", what, s->len, need);
  return UGHIP_OK;
}

// A matrix: F32 or BF16, and every matrix of a call like the first (*dtype < 0: not seen yet).
int check_w(const ughip_device* dev, const ughip_slice* s, size_t need, int* dtype, const char* what) {
  if (!s) return set_error(UGHIP_ERR_INVALID, "%s: null slice", what);
  if (s->dev != dev) return set_error(UGHIP_ERR_INVALID, "%s: slice lives on another device", what);
  if (s->dtype != UGHIP_F32 && s->dtype != UGHIP_BF16)
    return set_error(UGHIP_ERR_UNSUPPORTED, "%s: dtype %s, matrices are taken as F32 or BF16", what, dtype_name(s->dtype));
  if (*dtype >= 0 && s->dtype != *dtype) return set_error(UGHIP_ERR_INVALID, "%s: the matrices of one call must share a dtype", what);
  *dtype = s->dtype;
  if (s->len < need) return set_error(UGHIP_ERR_BOUNDS, "%s: slice has %zu elements, op needs %zu", what, s->len, need);
  return UGHIP_OK;
}

int check_k(size_t k, const char* what) {
  if (k == 0 || k % 4 != 0) return set_error(UGHIP_ERR_UNSUPPORTED, "%s: k = %zu is not a positive multiple of 4", what, k);
  if (k > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "%s: k = %zu is too large", what, k);
  return UGHIP_OK;
}

}  // namespace

extern "C" {

namespace {
// alpha == nullptr: no norm.  Otherwise the row has to fit the registers of the RMS kernels.
int check_rms(const ughip_device* dev, const ughip_slice* alpha, size_t k, const char* what) {
  if (!alpha) return UGHIP_OK;
  if (k > (size_t)256 * RMS_SLABS) return set_error(UGHIP_ERR_UNSUPPORTED, "%s: rows of %zu elements, the fused norm is built for up to %d", what, k, 256 * RMS_SLABS);
  return check(dev, alpha, k, what);
}
}  // namespace

int ughip_gemv_multi(ughip_device* dev, const ughip_slice* x, size_t n_mats, const ughip_slice* const* w, const size_t* n, size_t k, ughip_slice* dst) {
  return ughip_rms_gemv_multi(dev, x, nullptr, 0.f, n_mats, w, n, k, dst);
}

int ughip_rms_gemv_multi(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps, size_t n_mats, const ughip_slice* const* w,
                         const size_t* n, size_t k, ughip_slice* dst) {
  if (!dev || !w || !n) return set_error(UGHIP_ERR_INVALID, "gemv_multi: null argument");
  if (int rc = check_rms(dev, alpha, k, "gemv_multi alpha")) return rc;
  if (n_mats == 0 || n_mats > 3) return set_error(UGHIP_ERR_INVALID, "gemv_multi: %zu matrices, 1 to 3 are supported", n_mats);
  if (int rc = check_k(k, "gemv_multi")) return rc;
  if (int rc = check(dev, x, k, "gemv_multi x")) return rc;
  size_t total = 0;
  for (size_t i = 0; i < n_mats; ++i) total += n[i];
  if (total > 0x7fffffffull / 4) return set_error(UGHIP_ERR_INVALID, "gemv_multi: too many columns");
  if (int rc = check(dev, dst, total, "gemv_multi dst")) return rc;
  if (dst == x) return set_error(UGHIP_ERR_INVALID, "gemv_multi: dst aliases x");
  FusedArgs a{};
  a.x = static_cast<const float*>(x->ptr);
  a.k = (int)k;
  a.alpha = alpha ? static_cast<const float*>(alpha->ptr) : nullptr;
  a.eps = eps;
  size_t first = 0;
  int wdt = -1;
  for (size_t i = 0; i < 3; ++i) {
    if (i < n_mats) {
      if (int rc = check_w(dev, w[i], n[i] * k, &wdt, "gemv_multi w")) return rc;
      if (dst == w[i]) return set_error(UGHIP_ERR_INVALID, "gemv_multi: dst aliases a matrix");
      a.w[i] = w[i]->ptr;
      a.y[i] = static_cast<float*>(dst->ptr) + first;
      first += n[i];
    }
    a.col_end[i] = (int)first;
  }
  a.n_cols = (int)total;
  if (total == 0) return UGHIP_OK;
  if (int rc = device_activate(dev)) return rc;
  UGHIP_HIPCHK(launch<MODE_MULTI>(dev->stream, a, wdt));
  return UGHIP_OK;
}

int ughip_gemv_gate_up(ughip_device* dev, const ughip_slice* x, const ughip_slice* w_gate, const ughip_slice* w_up, ughip_slice* dst, size_t n, size_t k) {
  return ughip_rms_gemv_gate_up(dev, x, nullptr, 0.f, w_gate, w_up, dst, n, k);
}

int ughip_rms_gemv_gate_up(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps, const ughip_slice* w_gate, const ughip_slice* w_up,
                           ughip_slice* dst, size_t n, size_t k) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "gemv_gate_up: null device");
  if (int rc = check_rms(dev, alpha, k, "gemv_gate_up alpha")) return rc;
  if (int rc = check_k(k, "gemv_gate_up")) return rc;
  if (n > 0x7fffffffull / 4) return set_error(UGHIP_ERR_INVALID, "gemv_gate_up: too many columns");
  if (int rc = check(dev, x, k, "gemv_gate_up x")) return rc;
  int wdt = -1;
  if (int rc = check_w(dev, w_gate, n * k, &wdt, "gemv_gate_up gate")) return rc;
  if (int rc = check_w(dev, w_up, n * k, &wdt, "gemv_gate_up up")) return rc;
  if (int rc = check(dev, dst, n, "gemv_gate_up dst")) return rc;
  if (dst == x || dst == w_gate || dst == w_up) return set_error(UGHIP_ERR_INVALID, "gemv_gate_up: dst aliases an input");
  if (n == 0) return UGHIP_OK;
  FusedArgs a{};
  a.x = static_cast<const float*>(x->ptr);
  a.w[0] = w_gate->ptr;
  a.w[1] = w_up->ptr;
  a.alpha = alpha ? static_cast<const float*>(alpha->ptr) : nullptr;
  a.eps = eps;
  a.y[0] = static_cast<float*>(dst->ptr);
  a.col_end[0] = a.col_end[1] = a.col_end[2] = a.n_cols = (int)n;
  a.k = (int)k;
  if (int rc = device_activate(dev)) return rc;
  UGHIP_HIPCHK(launch<MODE_GATE_UP>(dev->stream, a, wdt));
  return UGHIP_OK;
}

int ughip_gemv_add(ughip_device* dev, const ughip_slice* x, const ughip_slice* w, const ughip_slice* residual, ughip_slice* dst, size_t n, size_t k) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "gemv_add: null device");
  if (int rc = check_k(k, "gemv_add")) return rc;
  if (n > 0x7fffffffull / 4) return set_error(UGHIP_ERR_INVALID, "gemv_add: too many columns");
  if (int rc = check(dev, x, k, "gemv_add x")) return rc;
  int wdt = -1;
  if (int rc = check_w(dev, w, n * k, &wdt, "gemv_add w")) return rc;
  if (int rc = check(dev, residual, n, "gemv_add residual")) return rc;
  if (int rc = check(dev, dst, n, "gemv_add dst")) return rc;
  if (dst == x || dst == w || dst == residual) return set_error(UGHIP_ERR_INVALID, "gemv_add: dst aliases an input");
  if (n == 0) return UGHIP_OK;
  FusedArgs a{};
  a.x = static_cast<const float*>(x->ptr);
  a.w[0] = w->ptr;
  a.y[0] = static_cast<float*>(dst->ptr);
  a.col_end[0] = a.col_end[1] = a.col_end[2] = a.n_cols = (int)n;
  a.k = (int)k;
  a.residual = static_cast<const float*>(residual->ptr);
  if (int rc = device_activate(dev)) return rc;
  UGHIP_HIPCHK(launch<MODE_ADD>(dev->stream, a, wdt));
  return UGHIP_OK;
}

}  // extern "C"
