// ug-llama's five custom ops as hand-written gfx950 kernels (wave64, 128-bit accesses).
// Semantics follow the CPU implementations in ug-llama/src/cpu_ops.rs:6-167; all f32.
#include <hip/hip_runtime.h>

#include <algorithm>

#include <cstdint>

#include "internal.h"
#include "ughip.h"
#include "wave_ops.h"

using namespace ughip;

namespace {


// Reduction across the NW waves of a workgroup through LDS; every thread gets the result.
template <int NW, bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* lds) {
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  if (NW == 1) return v;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = lds[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = IS_MAX ? fmaxf(r, lds[i]) : r + lds[i];
  return r;
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---- custom_softmax (cpu_ops.rs:6-31) --------------------------------------------------------
// One workgroup of NW waves per row; the row lives in registers (V float4 per thread), so HBM
// sees one read and one write per element.  Requires n_cols % 4 == 0 and
// n_cols <= NW * 64 * 4 * V.
template <int NW, int V>
__global__ void __launch_bounds__(NW * 64) softmax_rows_reg(const float* __restrict__ src, float* __restrict__ dst, int n_cols) {
  __shared__ float lds[NW > 1 ? NW : 1];
  const size_t row = blockIdx.x;
  const float4* s4 = reinterpret_cast<const float4*>(src + row * n_cols);
  float4* d4 = reinterpret_cast<float4*>(dst + row * n_cols);
  const int n4 = n_cols >> 2;
  float4 x[V];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    int c = threadIdx.x + i * NW * 64;
    if (c < n4) {
      x[i] = s4[c];
      m = fmaxf(fmaxf(m, fmaxf(x[i].x, x[i].y)), fmaxf(x[i].z, x[i].w));
    }
  }
  m = block_reduce<NW, true>(m, lds);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    int c = threadIdx.x + i * NW * 64;
    if (c < n4) {
      x[i].x = expf(x[i].x - m);
      x[i].y = expf(x[i].y - m);
      x[i].z = expf(x[i].z - m);
      x[i].w = expf(x[i].w - m);
      s += (x[i].x + x[i].y) + (x[i].z + x[i].w);
    }
  }
  s = block_reduce<NW, false>(s, lds);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    int c = threadIdx.x + i * NW * 64;
    if (c < n4) {
      x[i].x /= s;
      x[i].y /= s;
      x[i].z /= s;
      x[i].w /= s;
      __builtin_nontemporal_store(f32x4{x[i].x, x[i].y, x[i].z, x[i].w}, reinterpret_cast<f32x4*>(d4 + c));  // nobody in this launch reads it
    }
  }
}

// Wave per row for short rows (4 rows per workgroup), any n_cols <= 64 * V.
template <int V>
__global__ void __launch_bounds__(256) softmax_rows_wave(const float* __restrict__ src, float* __restrict__ dst, int n_rows, int n_cols) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const int lane = threadIdx.x & 63;
  const float* s = src + (size_t)row * n_cols;
  float* d = dst + (size_t)row * n_cols;
  float x[V];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    int c = lane + i * 64;
    x[i] = c < n_cols ? s[c] : -INFINITY;
    m = fmaxf(m, x[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    int c = lane + i * 64;
    x[i] = c < n_cols ? expf(x[i] - m) : 0.f;
    sum += x[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    int c = lane + i * 64;
    if (c < n_cols) d[c] = x[i] / sum;
  }
}

// Wave per row with 128-bit accesses (4 rows per workgroup): n_cols % 4 == 0, n_cols <= 256 * V.
// No LDS and no barrier: both reductions stay inside the wave.
template <int V>
__global__ void __launch_bounds__(256) softmax_rows_wave_v4(const float* __restrict__ src, float* __restrict__ dst, int n_rows, int n_cols) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const int lane = threadIdx.x & 63, n4 = n_cols >> 2;
  const float4* s4 = reinterpret_cast<const float4*>(src + (size_t)row * n_cols);
  float4* d4 = reinterpret_cast<float4*>(dst + (size_t)row * n_cols);
  float4 x[V];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int c = lane + i * 64;
    x[i] = c < n4 ? s4[c] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    m = fmaxf(fmaxf(m, fmaxf(x[i].x, x[i].y)), fmaxf(x[i].z, x[i].w));
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    // columns past the row end hold -inf and contribute exp(-inf) = 0
    x[i].x = expf(x[i].x - m);
    x[i].y = expf(x[i].y - m);
    x[i].z = expf(x[i].z - m);
    x[i].w = expf(x[i].w - m);
    sum += (x[i].x + x[i].y) + (x[i].z + x[i].w);
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int c = lane + i * 64;
    if (c < n4) d4[c] = make_float4(x[i].x / sum, x[i].y / sum, x[i].z / sum, x[i].w / sum);
  }
}

// Wave per row, resident: `gridDim.x` workgroups of four waves stay on the chip and every wave walks rows wave, wave +
// n_waves, ...  The row lives in registers (V float4 per lane, n_cols % 4 == 0, n_cols <= 256 * V), both reductions stay
// inside the wave (no LDS, no barrier), and the loads of the wave's next row are issued before the arithmetic of the
// current one, so every lane keeps V 128-bit loads in flight through the reductions, the exponentials and the stores.
// Loads are ordinary, stores go past the cache (nontemporal loads cost 10-20 % here: 4096 x 1024 6.6 against 5.5 us).
template <int V>
__global__ void __launch_bounds__(256) softmax_rows_wave_stream(const float* __restrict__ src, float* __restrict__ dst, int n_rows, int n_cols) {
  const int n_waves = gridDim.x * 4, lane = threadIdx.x & 63, n4 = n_cols >> 2;
  int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  auto load = [&](f32x4(&x)[V], int r) {
    const f32x4* s4 = reinterpret_cast<const f32x4*>(src + (size_t)r * n_cols);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int c = lane + i * 64;
      x[i] = c < n4 ? s4[c] : f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }
  };
  auto finish = [&](f32x4(&x)[V], int r) {
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < V; ++i) m = fmaxf(fmaxf(m, fmaxf(x[i].x, x[i].y)), fmaxf(x[i].z, x[i].w));
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      // columns past the row end hold -inf and contribute exp(-inf) = 0
      x[i].x = expf(x[i].x - m);
      x[i].y = expf(x[i].y - m);
      x[i].z = expf(x[i].z - m);
      x[i].w = expf(x[i].w - m);
      sum += (x[i].x + x[i].y) + (x[i].z + x[i].w);
    }
    sum = wave_sum(sum);
    f32x4* d4 = reinterpret_cast<f32x4*>(dst + (size_t)r * n_cols);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int c = lane + i * 64;
      const f32x4 y{x[i].x / sum, x[i].y / sum, x[i].z / sum, x[i].w / sum};
      if (c < n4) __builtin_nontemporal_store(y, d4 + c);
    }
  };
  f32x4 a[V], b[V];
  load(a, row);
  while (true) {
    int next = row + n_waves;
    if (next < n_rows) load(b, next);
    finish(a, row);
    if (next >= n_rows) break;
    row = next;
    next = row + n_waves;
    if (next < n_rows) load(a, next);
    finish(b, row);
    if (next >= n_rows) break;
    row = next;
  }
}

// Any row length: three passes over the row (the re-reads hit L2 for rows of this size).
__global__ void __launch_bounds__(1024) softmax_rows_generic(const float* __restrict__ src, float* __restrict__ dst, int n_cols) {
  __shared__ float lds[16];
  const size_t row = blockIdx.x;
  const float* s = src + row * n_cols;
  float* d = dst + row * n_cols;
  float m = -INFINITY;
  for (int c = threadIdx.x; c < n_cols; c += 1024) m = fmaxf(m, s[c]);
  m = block_reduce<16, true>(m, lds);
  float sum = 0.f;
  for (int c = threadIdx.x; c < n_cols; c += 1024) {
    float e = expf(s[c] - m);
    d[c] = e;
    sum += e;
  }
  sum = block_reduce<16, false>(sum, lds);
  for (int c = threadIdx.x; c < n_cols; c += 1024) d[c] /= sum;
}

// ---- causal_mask (cpu_ops.rs:33-56) --------------------------------------------------------------
// dst[b, i1, i2] = i2 <= i1 ? src : -inf.  Fully masked float4s never touch src.
__global__ void __launch_bounds__(256) causal_mask_v4(const float* __restrict__ src, float* __restrict__ dst, size_t n4, int s1, int s2) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  const int s2q = s2 >> 2;
  const int i2 = (int)(g % s2q) << 2;
  const int i1 = (int)((g / s2q) % s1);
  float4 v;
  if (i2 > i1) {
    v = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  } else {
    v = reinterpret_cast<const float4*>(src)[g];
    if (i2 + 1 > i1) v.y = -INFINITY;
    if (i2 + 2 > i1) v.z = -INFINITY;
    if (i2 + 3 > i1) v.w = -INFINITY;
  }
  __builtin_nontemporal_store(f32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<f32x4*>(dst) + g);  // past the cache: nobody in this launch reads it
}

__global__ void __launch_bounds__(256) causal_mask_scalar(const float* __restrict__ src, float* __restrict__ dst, size_t n, int s1, int s2) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n) return;
  const int i2 = (int)(g % s2);
  const int i1 = (int)((g / s2) % s1);
  dst[g] = i2 <= i1 ? src[g] : -INFINITY;
}

// ---- rope (cpu_ops.rs:91-126) and rope_i (cpu_ops.rs:58-89) -------------------------------------------
// src/dst are [bh, t, d]; the tables are read at row pos[0] + i_t.  A position that would run
// past the table poisons the output with NaN instead of faulting.
template <int W>  // pairs per thread: 4 (float4 path) or 1
__global__ void __launch_bounds__(256) rope_kernel(const float* __restrict__ src, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                   const int* __restrict__ pos, float* __restrict__ dst, size_t n_groups, int t, int d,
                                                   size_t table_len) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n_groups) return;
  const int h = d >> 1;
  const int hq = h / W;
  const int i_d = (int)(g % hq) * W;
  const size_t bt = g / hq;  // flat (bh, t)
  const int i_t = (int)(bt % t);
  const long long p = pos[0];
  const size_t i1 = bt * d + i_d;
  const size_t i2 = i1 + h;
  const size_t ics = ((size_t)p + i_t) * h + i_d;
  const bool ok = p >= 0 && ics + W <= table_len;
  if (W == 4) {
    float4 x1 = *reinterpret_cast<const float4*>(src + i1);
    float4 x2 = *reinterpret_cast<const float4*>(src + i2);
    float4 c, s;
    if (ok) {
      c = *reinterpret_cast<const float4*>(cos_t + ics);
      s = *reinterpret_cast<const float4*>(sin_t + ics);
    } else {
      c = s = make_float4(NAN, NAN, NAN, NAN);
    }
    float4 o1 = make_float4(x1.x * c.x - x2.x * s.x, x1.y * c.y - x2.y * s.y, x1.z * c.z - x2.z * s.z, x1.w * c.w - x2.w * s.w);
    float4 o2 = make_float4(x1.x * s.x + x2.x * c.x, x1.y * s.y + x2.y * c.y, x1.z * s.z + x2.z * c.z, x1.w * s.w + x2.w * c.w);
    *reinterpret_cast<float4*>(dst + i1) = o1;
    *reinterpret_cast<float4*>(dst + i2) = o2;
  } else {
    float x1 = src[i1], x2 = src[i2];
    float c = ok ? cos_t[ics] : NAN, s = ok ? sin_t[ics] : NAN;
    dst[i1] = x1 * c - x2 * s;
    dst[i2] = x1 * s + x2 * c;
  }
}

template <int W>  // pairs per thread: 2 (float4 path) or 1
__global__ void __launch_bounds__(256) rope_i_kernel(const float* __restrict__ src, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                     const int* __restrict__ pos, float* __restrict__ dst, size_t n_groups, int t, int d,
                                                     size_t table_len) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n_groups) return;
  const int h = d >> 1;
  const size_t pair = g * W;             // flat pair index over [bh, t, d/2]
  const size_t chunk = (size_t)t * h;    // pairs per bh
  const size_t in_chunk = pair % chunk;  // == i_t * (d/2) + i_d  (cpu_ops.rs:74-80)
  const long long p = pos[0];
  const size_t ics = (size_t)p * h + in_chunk;
  const bool ok = p >= 0 && ics + W <= table_len;
  if (W == 2) {
    float4 x = reinterpret_cast<const float4*>(src)[g];
    float2 c, s;
    if (ok) {
      c = *reinterpret_cast<const float2*>(cos_t + ics);
      s = *reinterpret_cast<const float2*>(sin_t + ics);
    } else {
      c = s = make_float2(NAN, NAN);
    }
    float4 o = make_float4(x.x * c.x - x.y * s.x, x.x * s.x + x.y * c.x, x.z * c.y - x.w * s.y, x.z * s.y + x.w * c.y);
    reinterpret_cast<float4*>(dst)[g] = o;
  } else {
    float a = src[2 * pair], b = src[2 * pair + 1];
    float c = ok ? cos_t[ics] : NAN, s = ok ? sin_t[ics] : NAN;
    dst[2 * pair] = a * c - b * s;
    dst[2 * pair + 1] = a * s + b * c;
  }
}

// ---- cat (cpu_ops.rs:128-167) ----------------------------------------------------------------------------
template <typename VT, int W>
__global__ void __launch_bounds__(256) cat_kernel(const float* __restrict__ lhs, const float* __restrict__ rhs, float* __restrict__ dst, size_t n_groups,
                                                  size_t d2_l, size_t d2_r) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n_groups) return;
  const size_t d2 = (d2_l + d2_r) / W;
  const size_t i1 = g / d2;
  const size_t j = (g % d2) * W;
  const float* s = j < d2_l ? lhs + i1 * d2_l + j : rhs + i1 * d2_r + (j - d2_l);
  reinterpret_cast<VT*>(dst)[g] = *reinterpret_cast<const VT*>(s);
}

int check_f32(const ughip_slice* s, size_t need, const char* what) {
  if (!s) return set_error(UGHIP_ERR_INVALID, "%s: null slice", what);
  if (s->dtype != UGHIP_F32) return set_error(UGHIP_ERR_INVALID, "%s: unexpected dtype %s, expected F32", what, dtype_name(s->dtype));
  if (s->len < need) return set_error(UGHIP_ERR_BOUNDS, "%s: slice has %zu elements, op needs %zu", what, s->len, need);
  return UGHIP_OK;
}

unsigned blocks_for(size_t n, unsigned per_block) { return (unsigned)((n + per_block - 1) / per_block); }

// ---- greedy step ------------------------------------------------------------------------------------
// Largest value of a row and its index (the lowest index among equal values), and the largest of
// the rest: what the host loop of a greedy decoder computes from the logits it reads back.
struct Top2 {
  float best;
  int idx;
  float second;
};

__device__ __forceinline__ Top2 top2_merge(const Top2& a, const Top2& b) {
  const bool a_wins = a.best > b.best || (a.best == b.best && a.idx < b.idx);
  Top2 r;
  r.best = a_wins ? a.best : b.best;
  r.idx = a_wins ? a.idx : b.idx;
  r.second = a_wins ? fmaxf(a.second, b.best) : fmaxf(b.second, a.best);
  return r;
}

__device__ __forceinline__ void top2_take(Top2& t, float v, int i) {
  if (v > t.best) {  // indices grow within a thread: an equal value never replaces an earlier one
    t.second = t.best;
    t.best = v;
    t.idx = i;
  } else if (v > t.second) {
    t.second = v;
  }
}

// VEC: the row starts on a 16-byte boundary; eight 128-bit loads per thread are in flight at once
// (a 32000-wide row is one trip), the last n % 4 elements are taken one by one.
template <bool VEC>
__global__ void __launch_bounds__(1024) argmax_row_kernel(const float* __restrict__ x, int n, int* __restrict__ token, int* __restrict__ ids,
                                                          float* __restrict__ vals, size_t slot) {
  __shared__ Top2 part[16];
  Top2 t{-INFINITY, 0x7fffffff, -INFINITY};
  if (VEC) {
    typedef float v4 __attribute__((ext_vector_type(4)));
    const int n4 = n >> 2;
    for (int i0 = threadIdx.x; i0 < n4; i0 += 8 * 1024) {
      v4 r[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) r[u] = reinterpret_cast<const v4*>(x)[min(i0 + u * 1024, n4 - 1)];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * 1024;
        if (i < n4) {
          top2_take(t, r[u].x, 4 * i);
          top2_take(t, r[u].y, 4 * i + 1);
          top2_take(t, r[u].z, 4 * i + 2);
          top2_take(t, r[u].w, 4 * i + 3);
        }
      }
    }
    for (int i = 4 * n4 + threadIdx.x; i < n; i += 1024) top2_take(t, x[i], i);
  } else {
    for (int i = threadIdx.x; i < n; i += 1024) top2_take(t, x[i], i);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Top2 u;
    u.best = __shfl_xor(t.best, o, 64);
    u.idx = __shfl_xor(t.idx, o, 64);
    u.second = __shfl_xor(t.second, o, 64);
    t = top2_merge(t, u);
  }
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) {
    Top2 r = part[0];
    for (int w = 1; w < 16; ++w) r = top2_merge(r, part[w]);
    if (r.idx == 0x7fffffff) r.idx = 0;  // a row of NaN / -inf only
    if (token) token[0] = r.idx;
    ids[slot] = r.idx;
    vals[2 * slot] = r.best;
    vals[2 * slot + 1] = r.second;
  }
}

}  // namespace

extern "C" {

int ughip_softmax_rows(ughip_device* dev, const ughip_slice* src, ughip_slice* dst, size_t n_rows, size_t n_cols) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (int rc = check_f32(src, n_rows * n_cols, "softmax src")) return rc;
  if (int rc = check_f32(dst, n_rows * n_cols, "softmax dst")) return rc;
  if (src == dst) return set_error(UGHIP_ERR_INVALID, "softmax: src and dst alias");
  if (n_rows == 0 || n_cols == 0) return UGHIP_OK;
  if (n_rows > 0x7fffffffull || n_cols > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "softmax: shape too large");
  if (int rc = device_activate(dev)) return rc;
  const float* s = static_cast<const float*>(src->ptr);
  float* d = static_cast<float*>(dst->ptr);
  hipStream_t st = dev->stream;
  const int nc = (int)n_cols, nr = (int)n_rows;
  // Rows of up to 2048 columns, at least 2048 of them and up to ~100 MB of traffic: one wave per row on at most 2048
  // workgroups (every wave slot of the chip), the loads of a wave's next row issued before the arithmetic of the current one.
  // Measured against the kernels below, us: 4096 x 512 3.97 / 4.47, x 768 5.04 / 6.25, x 1024 5.55 / 7.15, x 1536 7.5 / 7.98,
  // x 2048 9.0 / 10.6; 16384 x 512 9.6 / 11.3.  Larger problems walk too many rows per wave for that to win (16384 x 2048:
  // 42.1 against 38.4; 131072 x 1024: 191 against 179) and keep a fresh workgroup per row (or four rows).  Every kernel stores
  // past the cache: nobody in the launch reads the result (block per row, 2048 x 2048: 7.2 -> 5.4 us; 32768 x 4096: 178 -> 173).
  // SOFTMAX_STREAM (tuning aid): 0 never takes the resident kernel, n > 0 forces it onto n workgroups where it applies.
  long long stream = -1;
  tune_get(TUNE_SOFTMAX_STREAM, &stream);
  const bool stream_fits = n_cols % 4 == 0 && n_cols <= 8192;
  const bool stream_pays = n_cols % 4 == 0 && n_cols > 256 && n_cols <= 2048 && n_rows >= 2048 && n_rows * n_cols <= (3u << 22);
  if (stream_fits && (stream > 0 || (stream < 0 && stream_pays))) {
    const unsigned g = (unsigned)std::min<size_t>(stream > 0 ? (size_t)stream : 2048, blocks_for(n_rows, 4));
    if (n_cols <= 256) softmax_rows_wave_stream<1><<<g, 256, 0, st>>>(s, d, nr, nc);
    else if (n_cols <= 512) softmax_rows_wave_stream<2><<<g, 256, 0, st>>>(s, d, nr, nc);
    else if (n_cols <= 1024) softmax_rows_wave_stream<4><<<g, 256, 0, st>>>(s, d, nr, nc);
    else if (n_cols <= 2048) softmax_rows_wave_stream<8><<<g, 256, 0, st>>>(s, d, nr, nc);
    else if (n_cols <= 4096) softmax_rows_wave_stream<16><<<g, 256, 0, st>>>(s, d, nr, nc);
    else softmax_rows_wave_stream<32><<<g, 256, 0, st>>>(s, d, nr, nc);
  } else if (n_cols % 4 == 0 && n_cols <= 256) {
    softmax_rows_wave_v4<1><<<blocks_for(n_rows, 4), 256, 0, st>>>(s, d, nr, nc);
  } else if (n_cols % 4 == 0 && n_cols <= 512) {
    softmax_rows_wave_v4<2><<<blocks_for(n_rows, 4), 256, 0, st>>>(s, d, nr, nc);
  } else if (n_cols % 4 == 0 && n_cols <= 1024 && n_rows >= 2048) {
    softmax_rows_wave_v4<4><<<blocks_for(n_rows, 4), 256, 0, st>>>(s, d, nr, nc);
  } else if (n_cols <= 256) {
    softmax_rows_wave<4><<<blocks_for(n_rows, 4), 256, 0, st>>>(s, d, nr, nc);
  } else if (n_cols % 4 != 0 || n_cols > 16384) {
    softmax_rows_generic<<<nr, 1024, 0, st>>>(s, d, nc);
  } else if (n_cols <= 1024) {
    softmax_rows_reg<4, 1><<<nr, 256, 0, st>>>(s, d, nc);
  } else if (n_cols <= 2048) {
    softmax_rows_reg<4, 2><<<nr, 256, 0, st>>>(s, d, nc);
  } else if (n_cols <= 4096) {
    softmax_rows_reg<8, 2><<<nr, 512, 0, st>>>(s, d, nc);
  } else if (n_cols <= 8192) {
    softmax_rows_reg<16, 2><<<nr, 1024, 0, st>>>(s, d, nc);
  } else {
    softmax_rows_reg<16, 4><<<nr, 1024, 0, st>>>(s, d, nc);
  }
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_causal_mask(ughip_device* dev, const ughip_slice* src, ughip_slice* dst, size_t bh, size_t s1, size_t s2) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  const size_t n = bh * s1 * s2;
  if (int rc = check_f32(src, n, "causal_mask src")) return rc;
  if (int rc = check_f32(dst, n, "causal_mask dst")) return rc;
  if (src == dst) return set_error(UGHIP_ERR_INVALID, "causal_mask: src and dst alias");
  if (n == 0) return UGHIP_OK;
  if (s1 > 0x7fffffffull || s2 > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "causal_mask: shape too large");
  if (int rc = device_activate(dev)) return rc;
  const float* s = static_cast<const float*>(src->ptr);
  float* d = static_cast<float*>(dst->ptr);
  if (s2 % 4 == 0)
    causal_mask_v4<<<blocks_for(n / 4, 256), 256, 0, dev->stream>>>(s, d, n / 4, (int)s1, (int)s2);
  else
    causal_mask_scalar<<<blocks_for(n, 256), 256, 0, dev->stream>>>(s, d, n, (int)s1, (int)s2);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_rope(ughip_device* dev, const ughip_slice* src, const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos,
               ughip_slice* dst, size_t bh, size_t t, size_t d, int interleaved) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  const size_t n = bh * t * d;
  if (d % 2 != 0) return set_error(UGHIP_ERR_INVALID, "rope: head dim %zu is odd", d);
  if (int rc = check_f32(src, n, "rope src")) return rc;
  if (int rc = check_f32(dst, n, "rope dst")) return rc;
  if (int rc = check_f32(cos, t * d / 2, "rope cos")) return rc;
  if (int rc = check_f32(sin, t * d / 2, "rope sin")) return rc;
  if (!pos || pos->dtype != UGHIP_I32 || pos->len < 1) return set_error(UGHIP_ERR_INVALID, "rope: pos must be a non-empty I32 slice");
  if (src == dst) return set_error(UGHIP_ERR_INVALID, "rope: src and dst alias");
  if (n == 0) return UGHIP_OK;
  if (t > 0x7fffffffull || d > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "rope: shape too large");
  if (int rc = device_activate(dev)) return rc;
  const float* s = static_cast<const float*>(src->ptr);
  const float* c = static_cast<const float*>(cos->ptr);
  const float* sn = static_cast<const float*>(sin->ptr);
  const int* p = static_cast<const int*>(pos->ptr);
  float* o = static_cast<float*>(dst->ptr);
  const size_t table_len = cos->len < sin->len ? cos->len : sin->len;
  const size_t pairs = n / 2;
  if (!interleaved) {
    if ((d / 2) % 4 == 0)
      rope_kernel<4><<<blocks_for(pairs / 4, 256), 256, 0, dev->stream>>>(s, c, sn, p, o, pairs / 4, (int)t, (int)d, table_len);
    else
      rope_kernel<1><<<blocks_for(pairs, 256), 256, 0, dev->stream>>>(s, c, sn, p, o, pairs, (int)t, (int)d, table_len);
  } else {
    if ((d / 2) % 2 == 0)
      rope_i_kernel<2><<<blocks_for(pairs / 2, 256), 256, 0, dev->stream>>>(s, c, sn, p, o, pairs / 2, (int)t, (int)d, table_len);
    else
      rope_i_kernel<1><<<blocks_for(pairs, 256), 256, 0, dev->stream>>>(s, c, sn, p, o, pairs, (int)t, (int)d, table_len);
  }
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_cat(ughip_device* dev, const ughip_slice* lhs, const ughip_slice* rhs, ughip_slice* dst, size_t d1, size_t d2_l, size_t d2_r) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (int rc = check_f32(lhs, d1 * d2_l, "cat lhs")) return rc;
  if (int rc = check_f32(rhs, d1 * d2_r, "cat rhs")) return rc;
  const size_t n = d1 * (d2_l + d2_r);
  if (int rc = check_f32(dst, n, "cat dst")) return rc;
  if (dst == lhs || dst == rhs) return set_error(UGHIP_ERR_INVALID, "cat: dst aliases an input");
  if (n == 0) return UGHIP_OK;
  if (int rc = device_activate(dev)) return rc;
  const float* l = static_cast<const float*>(lhs->ptr);
  const float* r = static_cast<const float*>(rhs->ptr);
  float* o = static_cast<float*>(dst->ptr);
  if (d2_l % 4 == 0 && d2_r % 4 == 0)
    cat_kernel<float4, 4><<<blocks_for(n / 4, 256), 256, 0, dev->stream>>>(l, r, o, n / 4, d2_l, d2_r);
  else
    cat_kernel<float, 1><<<blocks_for(n, 256), 256, 0, dev->stream>>>(l, r, o, n, d2_l, d2_r);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_argmax_row(ughip_device* dev, const ughip_slice* logits, size_t n, size_t row, ughip_slice* token, ughip_slice* ids, ughip_slice* vals, size_t slot) {
  if (!dev || !logits || !ids || !vals) return set_error(UGHIP_ERR_INVALID, "argmax_row: null argument");
  if (logits->dtype != UGHIP_F32 || vals->dtype != UGHIP_F32 || ids->dtype != UGHIP_I32 || (token && token->dtype != UGHIP_I32))
    return set_error(UGHIP_ERR_INVALID, "argmax_row: expected F32 logits and values, I32 token and ids");
  if (n == 0 || n > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "argmax_row: row length %zu", n);
  if (logits->len < (row + 1) * n) return set_error(UGHIP_ERR_BOUNDS, "argmax_row: row %zu of %zu elements is outside a slice of %zu", row, n, logits->len);
  if (ids->len <= slot || vals->len < 2 * (slot + 1) || (token && token->len < 1))
    return set_error(UGHIP_ERR_BOUNDS, "argmax_row: slot %zu is outside the record slices", slot);
  if (int rc = device_activate(dev)) return rc;
  const float* x = static_cast<const float*>(logits->ptr) + row * n;
  int* tp = token ? static_cast<int*>(token->ptr) : nullptr;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0 && n >= 4)
    argmax_row_kernel<true><<<1, 1024, 0, dev->stream>>>(x, (int)n, tp, static_cast<int*>(ids->ptr), static_cast<float*>(vals->ptr), slot);
  else
    argmax_row_kernel<false><<<1, 1024, 0, dev->stream>>>(x, (int)n, tp, static_cast<int*>(ids->ptr), static_cast<float*>(vals->ptr), slot);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

}  // extern "C"
