// Attention fusions for gfx950 that go one step past the reference's op set (f32):
//
//   ughip_causal_softmax_rows  = causal_mask followed by custom_softmax (cpu_ops.rs:33-56, 6-31)
//                                in one pass: masked columns are never read and come out as 0.
//   ughip_attention_decode     = for one query position, the chain of ug-llama/src/model.rs:231-244
//                                repeat(k), repeat(v), q x k^T, * scale, softmax, x v
//                                in one launch, reading each K/V head once (no repeated copies).
//   ughip_rope_append          = for one new position, split/transpose + rope (or nothing) + cat
//                                (model.rs:213-230): the cache grows by one rotated row per head.
//   ughip_attention_decode with a rope table = the same with rope applied to q first, q and the
//                                result in the flat [b, nh * d] layout the projections use.
//
// All reduce in a fixed order (no atomics): results do not change from run to run.
#include <hip/hip_runtime.h>

#include "bf16_split.h"
#include "internal.h"
#include "ughip.h"
#include "wave_ops.h"

using namespace ughip;

namespace {


// All threads of a 256-thread workgroup get the max / the sum of v.
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce_256(float v, float* lds4) {
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
  __syncthreads();
  const float a = lds4[0], b = lds4[1], c = lds4[2], d = lds4[3];
  return IS_MAX ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
}

// ---- causal softmax -------------------------------------------------------------------------
// Rows of [bh, s1, s2]; row r keeps columns 0 .. r % s1.  Wave per row, 128-bit accesses:
// n_cols % 4 == 0 and n_cols <= 256 * V.
template <int V>
__global__ void __launch_bounds__(256) causal_softmax_wave_v4(const float* __restrict__ src, float* __restrict__ dst, int n_rows, int s1, int n_cols) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const int lane = threadIdx.x & 63, n4 = n_cols >> 2;
  const int lim = min(n_cols, row % s1 + 1);  // columns kept
  const float4* s4 = reinterpret_cast<const float4*>(src + (size_t)row * n_cols);
  float4* d4 = reinterpret_cast<float4*>(dst + (size_t)row * n_cols);
  float4 x[V];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int c = (lane + i * 64) * 4;
    x[i] = c < lim ? s4[lane + i * 64] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    if (c + 1 >= lim) x[i].y = -INFINITY;
    if (c + 2 >= lim) x[i].z = -INFINITY;
    if (c + 3 >= lim) x[i].w = -INFINITY;
    m = fmaxf(fmaxf(m, fmaxf(x[i].x, x[i].y)), fmaxf(x[i].z, x[i].w));
  }
  m = wave_max(m);  // column 0 is always kept: m is finite unless the data is not
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
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
    if (c < n4) {
      typedef float f32x4 __attribute__((ext_vector_type(4)));
      __builtin_nontemporal_store(f32x4{x[i].x / sum, x[i].y / sum, x[i].z / sum, x[i].w / sum}, reinterpret_cast<f32x4*>(d4 + c));  // past the cache
    }
  }
}

// Any row length: one workgroup per row, the kept part of the row is read twice.
__global__ void __launch_bounds__(256) causal_softmax_generic(const float* __restrict__ src, float* __restrict__ dst, int s1, int n_cols) {
  __shared__ float lds4[4];
  const size_t row = blockIdx.x;
  const int lim = min(n_cols, (int)(row % s1) + 1);
  const float* s = src + row * n_cols;
  float* d = dst + row * n_cols;
  float m = -INFINITY;
  for (int c = threadIdx.x; c < lim; c += 256) m = fmaxf(m, s[c]);
  m = block_reduce_256<true>(m, lds4);
  float sum = 0.f;
  for (int c = threadIdx.x; c < lim; c += 256) sum += expf(s[c] - m);
  sum = block_reduce_256<false>(sum, lds4);
  for (int c = threadIdx.x; c < n_cols; c += 256) d[c] = c < lim ? expf(s[c] - m) / sum : 0.f;
}

// ---- single-query attention -----------------------------------------------------------------------
// One workgroup of 1024 threads per query head.  q: [b, nh, d]; k, v: [b, nkv, s, d] (heads
// kv_head_stride elements apart: s * d, or capacity * d for a preallocated cache); dst: [b, nh, d].
// LPK = d / 4 lanes share one key row (one 128-bit load each, a row is one contiguous 4*d bytes);
// 1024 / LPK keys are in flight per step and four steps per loop trip, keys and values together,
// because at batch 1 this kernel is a chain of memory round trips and barriers, not a bandwidth
// problem: softmax runs in one pass with a running maximum per wave, and the only workgroup-wide
// exchange is the merge of the 16 waves at the end.
// With a rope table (cos_t != nullptr) q is rotated first, at table row pos[0] (rope: pairs
// (i, i + d/2); rope_i: pairs (2i, 2i + 1); cpu_ops.rs:58-126 for t = 1).
constexpr int ATT_THREADS = 1024, ATT_WAVES = ATT_THREADS / 64;
typedef float att_f32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(ATT_THREADS) attention_decode_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                                                       float* __restrict__ dst, int nh, int nkv, int s, size_t kv_head_stride,
                                                                       size_t q_batch_stride, int d, float scale, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                       const int* __restrict__ pos, size_t table_len, int interleaved,
                                                                       const float* __restrict__ k_new, const float* __restrict__ v_new, float* __restrict__ k_out,
                                                                       float* __restrict__ v_out, int nsplit, float* __restrict__ part) {
  __shared__ __attribute__((aligned(16))) float sc[ATT_WAVES * 64 * 4];  // one float4 per lane slot of every wave for the final merge
  __shared__ float wave_m[ATT_WAVES], wave_l[ATT_WAVES];
  __shared__ __attribute__((aligned(16))) float qs[256];
  __shared__ __attribute__((aligned(16))) float kn[256];
  __shared__ __attribute__((aligned(16))) float vn[256];
  const int tid = threadIdx.x;
  const int lpk = d >> 2, kpb = ATT_THREADS / lpk;  // lanes per key, keys per step
  const int c4 = tid % lpk, slot = tid / lpk;
  // nsplit > 1 (long caches): nsplit workgroups share a head, each takes a range of keys [j_lo, j_hi)
  // that is a whole number of loop trips and leaves its (maximum, sum, unnormalised row) in `part`
  // for attention_merge_kernel; one workgroup streams about 100 GB/s, so 32 heads alone cannot keep
  // up with a cache of thousands of rows.
  const int bh = blockIdx.x / nsplit, split = blockIdx.x % nsplit, b = bh / nh, h = bh % nh, kvh = h / (nh / nkv);
  const int chunk = nsplit == 1 ? s : (((s + nsplit - 1) / nsplit + 4 * kpb - 1) / (4 * kpb)) * (4 * kpb);
  const int j_lo = min(s, split * chunk), j_hi = min(s, j_lo + chunk);
  const float* qh = q + (size_t)b * q_batch_stride + (size_t)h * d;  // q_batch_stride = nh * d unless q is part of a wider row
  const float4* q4 = reinterpret_cast<const float4*>(qh);
  const float4* k4 = reinterpret_cast<const float4*>(k + ((size_t)b * nkv + kvh) * kv_head_stride);
  const float4* v4 = reinterpret_cast<const float4*>(v + ((size_t)b * nkv + kvh) * kv_head_stride);

  // k_new != nullptr: key / value row s-1 is not in the caches yet.  It comes from k_new / v_new
  // (rows of the same packed buffer as q: q_batch_stride apart, head kvh at kvh * d), the key is
  // rotated like q, and the first query head of every kv head stores both rows into the caches at
  // row s-1 for the steps to come (nobody reads that cache row in this launch).
  const float* knh = k_new ? k_new + (size_t)b * q_batch_stride + (size_t)kvh * d : nullptr;
  const float* vnh = k_new ? v_new + (size_t)b * q_batch_stride + (size_t)kvh * d : nullptr;
  const int j_new = k_new ? s - 1 : -1;
  // The cache rows of the first trip of both loops below (keys u * kpb + slot) are requested now:
  // they do not depend on pos or on the rotation, whose loads they overlap.
  // (native vectors: arrays of HIP's float4 struct are copied through memory)
  att_f32x4 kpre[4], vpre[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    // unconditional loads (a branch here sends the arrays to scratch memory): rows this lane has
    // no use for are read as row 0 and ignored below
    const int j = j_lo + u * kpb + slot;
    const size_t jj = j < j_hi && j != j_new ? (size_t)j : 0;
    kpre[u] = reinterpret_cast<const att_f32x4*>(k4)[jj * lpk + c4];
    vpre[u] = reinterpret_cast<const att_f32x4*>(v4)[jj * lpk + c4];
  }
  float4 qv;
  if (cos_t) {
    const int half = d >> 1;
    if (tid < 2 * half && (tid < half || k_new)) {
      const int pr = tid < half ? tid : tid - half;
      const float* src = tid < half ? qh : knh;
      float* out = tid < half ? qs : kn;
      const long long p = pos[0];
      const size_t ics = (size_t)p * half + pr;
      const bool ok = p >= 0 && ics < table_len;
      const float c = ok ? cos_t[ics] : NAN, sn = ok ? sin_t[ics] : NAN;
      const int i1 = interleaved ? 2 * pr : pr, i2 = interleaved ? 2 * pr + 1 : pr + half;
      const float x1 = src[i1], x2 = src[i2];
      out[i1] = x1 * c - x2 * sn;
      out[i2] = x1 * sn + x2 * c;
    }
    if (k_new && tid >= 512 && tid < 512 + d) vn[tid - 512] = vnh[tid - 512];
    __syncthreads();
    qv = reinterpret_cast<const float4*>(qs)[c4];
  } else {
    if (k_new && tid < d) kn[tid] = knh[tid];
    if (k_new && tid >= 512 && tid < 512 + d) vn[tid - 512] = vnh[tid - 512];
    if (k_new) __syncthreads();
    qv = q4[c4];
  }
  if (k_out && h % (nh / nkv) == 0 && split == 0 && tid < 2 * lpk) {
    const size_t row = (((size_t)b * nkv + kvh) * kv_head_stride + (size_t)(s - 1) * d) / 4;
    if (tid < lpk) reinterpret_cast<float4*>(k_out)[row + tid] = reinterpret_cast<const float4*>(kn)[tid];
    else reinterpret_cast<float4*>(v_out)[row + tid - lpk] = reinterpret_cast<const float4*>(vn)[tid - lpk];
  }
  // One pass over the keys, four key rows and four value rows per lane group in flight.  Every lane
  // group keeps a running maximum m_run, the sum l_run of exp(score - m_run) and the weighted value
  // rows acc of the keys it has seen (rescaled when the maximum moves): inside the loop nothing
  // crosses the group, so a long cache costs arithmetic, not exchanges.  The groups of a wave and
  // then the 16 waves are merged once at the end.  Scores and probabilities never leave registers.
  float m_run = -INFINITY, l_run = 0.f;
  att_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  auto load_rows = [&](const float4* base, int j0, att_f32x4 (&r)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * kpb + slot;
      const size_t jj = j < j_hi && j != j_new ? (size_t)j : 0;
      r[u] = reinterpret_cast<const att_f32x4*>(base)[jj * lpk + c4];
    }
  };
  auto trip = [&](int j0, const att_f32x4 (&kr)[4], const att_f32x4 (&vr)[4]) {
    float p[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * kpb + slot;
      const att_f32x4 kv = j == j_new ? reinterpret_cast<const att_f32x4*>(kn)[c4] : kr[u];
      p[u] = (qv.x * kv.x + qv.y * kv.y) + (qv.z * kv.z + qv.w * kv.w);
    }
    float mt = -INFINITY;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float pu = p[u];
      // sum over the lpk lanes of this key (a power of two <= 64); from 16 lanes up the last four
      // steps are rotations within rows of 16
      if (lpk >= 16) {
        if (lpk > 32) pu += __shfl_xor(pu, 32, 64);
        if (lpk > 16) pu += __shfl_xor(pu, 16, 64);
        pu = row_sum16(pu);
      } else {
        for (int o = lpk >> 1; o > 0; o >>= 1) pu += __shfl_xor(pu, o, 64);
      }
      p[u] = j0 + u * kpb + slot < j_hi ? pu * scale : -INFINITY;
      mt = fmaxf(mt, p[u]);
    }
    const float m_new = fmaxf(m_run, mt);
    // a group that has not seen a key yet keeps its zeros (exp(-inf - -inf) would be NaN)
    const float alpha = m_new == -INFINITY ? 0.f : expf(m_run - m_new);  // 0 on the group's first keys (m_run = -inf)
    acc *= alpha;
    float lt = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * kpb + slot;
      const float e = m_new == -INFINITY ? 0.f : expf(p[u] - m_new);  // 0 for the keys past the end
      const att_f32x4 vv = j == j_new ? reinterpret_cast<const att_f32x4*>(vn)[c4] : vr[u];
      acc += e * vv;
      lt += e;  // the lanes of a group all hold the same e and the same sums
    }
    l_run = l_run * alpha + lt;
    m_run = m_new;
  };
  trip(j_lo, kpre, vpre);
  for (int j0 = j_lo + 4 * kpb; j0 < j_hi; j0 += 4 * kpb) {
    att_f32x4 kr[4], vr[4];
    load_rows(k4, j0, kr);
    load_rows(v4, j0, vr);
    trip(j0, kr, vr);
  }
  // the groups of one wave (lanes lpk apart): bring them to the wave's maximum, then add up ...
  {
    float m_w = m_run;
    for (int o = lpk; o < 64; o <<= 1) m_w = fmaxf(m_w, __shfl_xor(m_w, o, 64));
    const float f = m_run == -INFINITY ? 0.f : expf(m_run - m_w);  // m_w is finite wherever m_run is
    acc *= f;
    l_run *= f;
    m_run = m_w;
  }
  for (int o = lpk; o < 64; o <<= 1) {
    l_run += __shfl_xor(l_run, o, 64);
    acc.x += __shfl_xor(acc.x, o, 64);
    acc.y += __shfl_xor(acc.y, o, 64);
    acc.z += __shfl_xor(acc.z, o, 64);
    acc.w += __shfl_xor(acc.w, o, 64);
  }
  // ... then the waves in order, each weighted by exp(its maximum - the overall one)
  att_f32x4* red = reinterpret_cast<att_f32x4*>(sc);
  const int lane = tid & 63, wave = tid >> 6;
  if (lane < lpk) red[wave * 64 + lane] = acc;
  if (lane == 0) {
    wave_m[wave] = m_run;
    wave_l[wave] = l_run;
  }
  __syncthreads();
  // Thread w * lpk + c weighs column group c of wave w; the 64 / lpk waves that share a wave of these threads are added
  // by a butterfly over the lanes lpk apart, the ATT_WAVES * lpk / 64 such sums by the first lpk threads in wave order: a
  // fixed order, and 16 times fewer instructions than one lane group walking all the waves.
  const int n_merge = ATT_WAVES * lpk;  // <= ATT_THREADS: lpk <= 64
  att_f32x4 o = {0.f, 0.f, 0.f, 0.f};
  float sum = 0.f, mx = -INFINITY;
  if (tid < n_merge) {
    mx = wave_m[0];  // the first key of the range belongs to wave 0: finite unless the range is empty or the data is not
#pragma unroll
    for (int w = 1; w < ATT_WAVES; ++w) mx = fmaxf(mx, wave_m[w]);
    const int w = tid / lpk, c = tid % lpk;
    const float f = wave_m[w] == -INFINITY ? 0.f : expf(wave_m[w] - mx);  // 0 for a wave without keys
    o = f * red[w * 64 + c];
    sum = f * wave_l[w];
    for (int off = lpk; off < 64; off <<= 1) {
      sum += __shfl_xor(sum, off, 64);
      o.x += __shfl_xor(o.x, off, 64);
      o.y += __shfl_xor(o.y, off, 64);
      o.z += __shfl_xor(o.z, off, 64);
      o.w += __shfl_xor(o.w, off, 64);
    }
  }
  __syncthreads();  // every partial has been read: the merge buffers are free for the second stage
  const int n_stage2 = (n_merge + 63) / 64;
  if (tid < n_merge && lane < lpk) {
    red[wave * 64 + lane] = o;
    if (lane == 0) wave_l[wave] = sum;
  }
  __syncthreads();
  if (tid < lpk) {
    o = red[tid];
    sum = wave_l[0];
    for (int w = 1; w < n_stage2; ++w) {
      o += red[w * 64 + tid];
      sum += wave_l[w];
    }
    if (nsplit == 1) {
      reinterpret_cast<att_f32x4*>(dst + (size_t)bh * d)[tid] = o / sum;
    } else {
      float* pp = part + ((size_t)bh * nsplit + split) * (size_t)(d + 4);
      if (tid == 0) {
        pp[0] = mx;
        pp[1] = sum;
      }
      reinterpret_cast<att_f32x4*>(pp + 4)[tid] = o;
    }
  }
}

// The ranges of one head put together: out = sum_i exp(m_i - M) o_i / sum_i exp(m_i - M) l_i, in range order.
__global__ void __launch_bounds__(64) attention_merge_kernel(const float* __restrict__ part, float* __restrict__ dst, int nsplit, int d) {
  // One trip to memory: lane i fetches the (maximum, sum) pair of range i while every lane already has the rows of the
  // first eight ranges for its four columns on their way; the factors reach the columns' lanes by lane reads.
  // nsplit <= 64 (the launcher's limit); ranges are folded in index order, the sum of the weights in the fixed
  // butterfly order of wave_sum.
  typedef float att_f32x2 __attribute__((ext_vector_type(2)));
  const int bh = blockIdx.x, t = threadIdx.x;
  const bool col = t < (d >> 2);
  const float* pp = part + (size_t)bh * nsplit * (size_t)(d + 4);
  att_f32x4 r[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = col && j < nsplit ? reinterpret_cast<const att_f32x4*>(pp + (size_t)j * (d + 4) + 4)[t] : att_f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  if (t < nsplit) {
    const att_f32x2 ml = *reinterpret_cast<const att_f32x2*>(pp + (size_t)t * (d + 4));
    m = ml.x, l = ml.y;
  }
  const float mx = ughip::wave_max(m);
  const float f = m == -INFINITY ? 0.f : expf(m - mx);  // 0 for a range without keys (and for lanes past the last range)
  const float sum = ughip::wave_sum(f * l);
  att_f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 8; ++j) o += __shfl(f, j, 64) * r[j];
  for (int i0 = 8; i0 < nsplit; i0 += 8) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      r[j] = col && i0 + j < nsplit ? reinterpret_cast<const att_f32x4*>(pp + (size_t)(i0 + j) * (d + 4) + 4)[t] : att_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; ++j) o += __shfl(f, (i0 + j) & 63, 64) * r[j];
  }
  if (col) reinterpret_cast<att_f32x4*>(dst + (size_t)bh * d)[t] = o / sum;
}

// ---- cache append for one new position ------------------------------------------------------------
// dst [bh, s_old + 1, d] = cat(cache [bh, s_old, d], row(x [bh, d])) along the middle dim, the new
// row rotated when a table is given.  One thread per float4 of dst (d % 8 == 0).
__global__ void __launch_bounds__(256) rope_append_kernel(const float* __restrict__ cache, const float* __restrict__ x, float* __restrict__ dst, size_t n4,
                                                          int s_old, int d, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                          const int* __restrict__ pos, size_t table_len, int interleaved) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  const int d4 = d >> 2;
  const int c4 = (int)(g % d4);
  const size_t row = g / d4;  // flat (bh, j), j in 0..s_old
  const int j = (int)(row % (s_old + 1));
  const size_t bh = row / (s_old + 1);
  float4 out;
  if (j < s_old) {
    out = reinterpret_cast<const float4*>(cache)[(bh * s_old + j) * d4 + c4];
  } else if (!cos_t) {
    out = reinterpret_cast<const float4*>(x)[bh * d4 + c4];
  } else {
    const float* xr = x + bh * d;
    const int half = d >> 1;
    const long long p = pos[0];
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = c4 * 4 + e;  // output element
      // pair index and whether i is the first or the second element of its pair
      const int pr = interleaved ? i >> 1 : (i < half ? i : i - half);
      const bool first = interleaved ? (i & 1) == 0 : i < half;
      const int i1 = interleaved ? 2 * pr : pr, i2 = interleaved ? 2 * pr + 1 : pr + half;
      const size_t ics = (size_t)p * half + pr;
      const bool ok = p >= 0 && ics < table_len;
      const float c = ok ? cos_t[ics] : NAN, sn = ok ? sin_t[ics] : NAN;
      const float x1 = xr[i1], x2 = xr[i2];
      o[e] = first ? x1 * c - x2 * sn : x1 * sn + x2 * c;
    }
    out = make_float4(o[0], o[1], o[2], o[3]);
  }
  reinterpret_cast<float4*>(dst)[g] = out;
}

// ---- cache append in place ------------------------------------------------------------------------
// cache [b, n, cap, d], x [b, t, n * d] (rows x_row_stride apart): cache[b, h, s_old + i, :] =
// x[b, i, h * d .. (h + 1) * d), rotated at table row pos[0] + i when a table is given.  One thread
// per float4 of x (d % 4 == 0).
__device__ __forceinline__ void kv_append_body(size_t g, float* __restrict__ cache, const float* __restrict__ x, size_t x_row_stride, int t, int n, int d,
                                               size_t cap, int s_old, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                               const int* __restrict__ pos, size_t table_len, int interleaved) {
  const int d4 = d >> 2;
  const int c4 = (int)(g % d4);
  size_t rest = g / d4;
  const int h = (int)(rest % n);
  rest /= n;
  const int i = (int)(rest % t);
  const size_t b = rest / t;
  const float* xr = x + (b * t + i) * x_row_stride + (size_t)h * d;  // x_row_stride = n * d unless x is part of a wider row
  float4 out;
  if (!cos_t) {
    out = reinterpret_cast<const float4*>(xr)[c4];
  } else {
    const int half = d >> 1;
    const long long p = (long long)pos[0] + i;
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = c4 * 4 + e;  // output element; its pair and whether it is the pair's first element
      const int pr = interleaved ? c >> 1 : (c < half ? c : c - half);
      const bool first = interleaved ? (c & 1) == 0 : c < half;
      const int i1 = interleaved ? 2 * pr : pr, i2 = interleaved ? 2 * pr + 1 : pr + half;
      const size_t ics = (size_t)p * half + pr;
      const bool ok = p >= 0 && ics < table_len;
      const float cs = ok ? cos_t[ics] : NAN, sn = ok ? sin_t[ics] : NAN;
      const float x1 = xr[i1], x2 = xr[i2];
      o[e] = first ? x1 * cs - x2 * sn : x1 * sn + x2 * cs;
    }
    out = make_float4(o[0], o[1], o[2], o[3]);
  }
  reinterpret_cast<float4*>(cache + ((b * n + h) * cap + (size_t)s_old + i) * d)[c4] = out;
}

__global__ void __launch_bounds__(256) kv_append_kernel(float* __restrict__ cache, const float* __restrict__ x, size_t x_row_stride, size_t n4, int t, int n,
                                                        int d, size_t cap, int s_old, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                        const int* __restrict__ pos, size_t table_len, int interleaved) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  kv_append_body(g, cache, x, x_row_stride, t, n, d, cap, s_old, cos_t, sin_t, pos, table_len, interleaved);
}

// Keys (blockIdx.y == 0, rotated when a table is given) and values (blockIdx.y == 1, copied) of the same new positions in one launch.
__global__ void __launch_bounds__(256) kv_append_pair_kernel(float* __restrict__ kcache, float* __restrict__ vcache, const float* __restrict__ xk,
                                                             const float* __restrict__ xv, size_t x_row_stride, size_t n4, int t, int n, int d, size_t cap,
                                                             int s_old, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                             const int* __restrict__ pos, size_t table_len, int interleaved) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n4) return;
  if (blockIdx.y == 0) kv_append_body(g, kcache, xk, x_row_stride, t, n, d, cap, s_old, cos_t, sin_t, pos, table_len, interleaved);
  else kv_append_body(g, vcache, xv, x_row_stride, t, n, d, cap, s_old, nullptr, nullptr, nullptr, 0, 0);
}

// ---- causal attention over a cache, many query positions ------------------------------------------
// q, dst: [b, t, nh * D] (q rows q_row_stride apart); k, v: [b, nkv, cap, D] with rows 0 .. s-1 valid.  Query i sits at position
// s - t + i and sees keys 0 .. s - t + i (model.rs:231-244 with the mask of cpu_ops.rs:33-56 moved to
// that offset).  Scores never reach memory: a group of 4 waves owns 32 queries of one head, its waves
// take every fourth block of 32 keys and keep a running (max, sum, output) per query, merged at the
// end in wave order.
//
// Everything is v_mfma_f32_32x32x2_f32 on transposed products, so that a lane owns ONE query
// (column lane % 32) and the softmax statistics never cross lanes except between the two halves:
//   S^T = K Q^T   (M = keys, N = queries, K = D): A = K[key = lane % 32][c], B = Q[query = lane % 32][c]
//                 with c = j for lanes 0-31 and D/2 + j for lanes 32-63 in MFMA j -- both operands are
//                 D/2 consecutive floats per lane, loaded once per block (K) or once per kernel (Q).
//   O^T = V^T P^T (M = D, N = queries, K = keys): accumulator register r of S^T holds key
//                 8 (r / 4) + 4 (lane / 32) + r % 4, which is exactly the pair of keys MFMA r consumes
//                 (lower half one key, upper half the other): P feeds back as the B operand without
//                 any data movement; A = V[that key][lane % 32 + 32 * block].
typedef float att_f32x16 __attribute__((ext_vector_type(16)));

// exp(x) for x <= 0 in six branch-free instructions: x log2(e) is formed as a rounded product t plus
// its exact remainder r (two FMAs, log2(e) split in two), then 2^t (1 + r ln 2).  Within 2 ulp over the
// range the exponentials of a softmax live in; anything below about -87 (ATT_MASKED included) gives 0.
constexpr float ATT_MASKED = -1e30f;
__device__ __forceinline__ float att_exp(float x) {
  constexpr float L2E_HI = 1.44269502162933349609375f, L2E_LO = 1.925963033500011e-8f, LN2 = 0.693147182464599609375f;
  const float t = x * L2E_HI;
  float r = __builtin_fmaf(x, L2E_HI, -t);
  r = __builtin_fmaf(x, L2E_LO, r);
  const float y = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(y, r * LN2, y);
}

template <int D, int GROUPS>
__global__ void __launch_bounds__(256 * GROUPS) attention_prefill_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                                                float* __restrict__ dst, int nh, int nkv, int t, int s, size_t cap,
                                                                size_t q_row_stride, float scale, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                const int* __restrict__ pos, size_t table_len, int interleaved) {
  constexpr int H = D / 2, DB = D / 32;  // floats of q / k per lane; 32-wide blocks of the head dimension
  // K / V blocks reach the MFMA operand layout through a staging area private to each wave: rows
  // are loaded from global memory whole (consecutive lanes, consecutive 16 bytes) and read back
  // one row per lane.  Row pitches of D + 4 (128-bit reads of 16 rows) and D + 8 (32-bit reads of
  // two rows 4 apart) floats keep both read patterns free of bank conflicts.
  constexpr int NV = D / 8, KP = D + 4, VP = D + 8, STAGE = 32 * (KP + VP);
  extern __shared__ __attribute__((aligned(16))) float smem[];
  // the merge buffers take the staging area over once every wave is out of its loop
  float (*merge_ml_all)[3][2][64] = reinterpret_cast<float (*)[3][2][64]>(smem);
  float (*merge_o_all)[3][DB * 16][64] = reinterpret_cast<float (*)[3][DB * 16][64]>(smem + GROUPS * 3 * 2 * 64);
  static_assert(GROUPS * (3 * 2 * 64 + 3 * DB * 16 * 64) <= 4 * GROUPS * STAGE, "merge buffers must fit the staging area");
  const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3, group = tid >> 8;
  float* const kst = smem + (size_t)(tid >> 6) * STAGE;
  float* const vst = kst + 32 * KP;
  const int col = lane & 31, hh = lane >> 5;
  const int bh = blockIdx.y, b = bh / nh, head = bh % nh, kvh = head / (nh / nkv);
  // GROUPS == 2: a workgroup takes the query blocks x and n - 1 - x, one per group of 4 waves, so
  // that under the causal mask every workgroup has the same number of key blocks to go through
  const int n_qb = (t + 31) / 32;
  const int qb = GROUPS == 1 ? n_qb - 1 - (int)blockIdx.x : (group == 0 ? n_qb - 1 - (int)blockIdx.x : (int)blockIdx.x);
  const bool idle = GROUPS == 2 && group == 1 && qb == n_qb - 1 - qb;  // odd count: the middle block belongs to group 0
  float (*merge_ml)[2][64] = merge_ml_all[group];
  float (*merge_o)[64] = merge_o_all[group][0];
  const int q0 = qb * 32;
  const int qi = min(q0 + col, t - 1);        // rows past t repeat the last query and are not stored
  const int q_pos = s - t + qi;               // last key this query sees
  const int last_pos = s - t + min(q0 + 31, t - 1);
  const int q_pos_min = s - t + min(q0, t - 1);  // the query of this block that sees the fewest keys
  const float* kb_ptr = k + ((size_t)b * nkv + kvh) * cap * D;
  const float* vb_ptr = v + ((size_t)b * nkv + kvh) * cap * D;

  // One block of 32 rows (rows past s repeat row s-1: they are masked, and a block index past
  // the end is harmless) as NV 128-bit loads per lane, and its way into the staging area.
  auto load_block = [&](const float* base, int kb, att_f32x4 (&raw)[NV]) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int f4 = i * 64 + lane, row = f4 / (D / 4), c4 = f4 % (D / 4);
      raw[i] = *reinterpret_cast<const att_f32x4*>(base + (size_t)min(kb * 32 + row, s - 1) * D + c4 * 4);
    }
  };
  auto stage_block = [&](float* dst_rows, int pitch, const att_f32x4 (&raw)[NV]) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int f4 = i * 64 + lane, row = f4 / (D / 4), c4 = f4 % (D / 4);
      *reinterpret_cast<att_f32x4*>(dst_rows + row * pitch + c4 * 4) = raw[i];
    }
  };

  // the first blocks are requested before the query row, whose table row hangs off a load of pos
  att_f32x4 kraw[NV], vraw[NV];
  load_block(kb_ptr, wave, kraw);
  load_block(vb_ptr, wave, vraw);

  // this lane's half of its (rotated) query row
  float qr[H];
  {
    const float* qrow = q + ((size_t)b * t + qi) * q_row_stride + (size_t)head * D;  // nh * D unless q is part of a wider row
    if (!cos_t) {
#pragma unroll
      for (int j = 0; j < H; j += 4) {
        const float4 x = *reinterpret_cast<const float4*>(qrow + hh * H + j);
        qr[j] = x.x, qr[j + 1] = x.y, qr[j + 2] = x.z, qr[j + 3] = x.w;
      }
    } else {
      // table row pos[0] + qi, read with 128-bit loads from a clamped address; a row outside the
      // table turns the query into NaN (what the bounds error of the op-by-op path would flag)
      const long long p = (long long)pos[0] + qi;
      const bool ok = p >= 0 && (size_t)(p + 1) * H <= table_len;
      const size_t row = ok ? (size_t)p * H : 0;
      if (interleaved) {
        // pairs (2i, 2i + 1): both elements and their table entry lie in this lane's half
        float xh[H], ch[H / 2], sh[H / 2];
#pragma unroll
        for (int j = 0; j < H; j += 4) {
          const float4 x = *reinterpret_cast<const float4*>(qrow + hh * H + j);
          xh[j] = x.x, xh[j + 1] = x.y, xh[j + 2] = x.z, xh[j + 3] = x.w;
        }
#pragma unroll
        for (int j = 0; j < H / 2; j += 4) {
          const float4 c = *reinterpret_cast<const float4*>(cos_t + row + hh * (H / 2) + j);
          const float4 sn = *reinterpret_cast<const float4*>(sin_t + row + hh * (H / 2) + j);
          ch[j] = c.x, ch[j + 1] = c.y, ch[j + 2] = c.z, ch[j + 3] = c.w;
          sh[j] = sn.x, sh[j + 1] = sn.y, sh[j + 2] = sn.z, sh[j + 3] = sn.w;
        }
#pragma unroll
        for (int j = 0; j < H; ++j) {
          const float x1 = xh[j & ~1], x2 = xh[j | 1], cs = ch[j >> 1], sn = sh[j >> 1];
          qr[j] = (j & 1) ? x1 * sn + x2 * cs : x1 * cs - x2 * sn;
        }
      } else {
        // pairs (i, i + D/2): the lower half of the lanes produces x1 c - x2 s, the upper x1 s + x2 c
        float xa[H], xb[H], ch[H], sh[H];
#pragma unroll
        for (int j = 0; j < H; j += 4) {
          const float4 a = *reinterpret_cast<const float4*>(qrow + j);
          const float4 bq = *reinterpret_cast<const float4*>(qrow + H + j);
          const float4 c = *reinterpret_cast<const float4*>(cos_t + row + j);
          const float4 sn = *reinterpret_cast<const float4*>(sin_t + row + j);
          xa[j] = a.x, xa[j + 1] = a.y, xa[j + 2] = a.z, xa[j + 3] = a.w;
          xb[j] = bq.x, xb[j + 1] = bq.y, xb[j + 2] = bq.z, xb[j + 3] = bq.w;
          ch[j] = c.x, ch[j + 1] = c.y, ch[j + 2] = c.z, ch[j + 3] = c.w;
          sh[j] = sn.x, sh[j + 1] = sn.y, sh[j + 2] = sn.z, sh[j + 3] = sn.w;
        }
#pragma unroll
        for (int j = 0; j < H; ++j) qr[j] = hh ? xa[j] * sh[j] + xb[j] * ch[j] : xa[j] * ch[j] - xb[j] * sh[j];
      }
      if (!ok) {
#pragma unroll
        for (int j = 0; j < H; ++j) qr[j] = NAN;
      }
    }
  }

  float m_run = ATT_MASKED, l_half = 0.f;  // l_half: sum over the keys this half of the query's lanes holds
  att_f32x16 o[DB];
#pragma unroll
  for (int e = 0; e < DB; ++e)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[e][r] = 0.f;

  const int n_blocks = idle ? 0 : last_pos / 32 + 1;
  // K and V of the next block are in flight (in registers) while this one is multiplied
  for (int kb = wave; kb < n_blocks; kb += 4) {
    const int key0 = kb * 32;
    stage_block(kst, KP, kraw);
    stage_block(vst, VP, vraw);
    load_block(kb_ptr, kb + 4, kraw);
    load_block(vb_ptr, kb + 4, vraw);
    __builtin_amdgcn_sched_barrier(0);  // keeps the loads up here instead of next to their uses
    // K operand: D/2 consecutive floats of key row col
    float kr[H];
#pragma unroll
    for (int j = 0; j < H; j += 4) {
      const att_f32x4 x = *reinterpret_cast<const att_f32x4*>(kst + col * KP + hh * H + j);
      kr[j] = x.x, kr[j + 1] = x.y, kr[j + 2] = x.z, kr[j + 3] = x.w;
    }
    att_f32x16 sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
    for (int j = 0; j < H; ++j) sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kr[j], qr[j], sc, 0, 0, 0);
    // V operand of MFMA r: row 8 (r / 4) + 4 hh + r % 4 of the block, column col + 32 e.  Requested
    // while the score MFMAs run, first needed after the exponentials.
    float vr[DB][16];
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int r = 0; r < 16; ++r) vr[e][r] = vst[((r >> 2) * 8 + hh * 4 + (r & 3)) * VP + e * 32 + col];
    __builtin_amdgcn_sched_barrier(0);
    // masked scores become ATT_MASKED, a finite stand-in for -inf that the exponential below maps to 0
    float mx = ATT_MASKED;
    if (key0 + 31 > q_pos_min) {  // wave-uniform: only blocks that touch the diagonal have anything to mask
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + (r >> 2) * 8 + hh * 4 + (r & 3);
        sc[r] = key <= q_pos ? sc[r] * scale : ATT_MASKED;
        mx = fmaxf(mx, sc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sc[r] *= scale;
        mx = fmaxf(mx, sc[r]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new <= ATT_MASKED ? 0.f : m_new;  // no key seen yet: every exponential below is 0
    const float alpha = att_exp(m_run - m_use);
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = att_exp(sc[r] - m_use);
      psum += sc[r];
    }
    l_half = l_half * alpha + psum;
    if (__any(alpha != 1.f)) {  // the running maximum settles after a few blocks
#pragma unroll
      for (int e = 0; e < DB; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[e][r] *= alpha;
    }
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[e][r], sc[r], o[e], 0, 0, 0);
    __builtin_amdgcn_wave_barrier();  // the next trip overwrites the staging area
  }
  __syncthreads();  // every wave is done with its staging area: the merge buffers may take it over

  // merge the four waves' partial results in wave order
  if (wave != 0) {
    merge_ml[wave - 1][0][lane] = m_run;
    merge_ml[wave - 1][1][lane] = l_half;
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int r = 0; r < 16; ++r) merge_o[(wave - 1) * DB * 16 + e * 16 + r][lane] = o[e][r];
  }
  __syncthreads();
  if (wave != 0 || idle) return;
  float m_tot = m_run;
#pragma unroll
  for (int w = 0; w < 3; ++w) m_tot = fmaxf(m_tot, merge_ml[w][0][lane]);
  // key 0 is visible to every query and belongs to wave 0's first block: m_tot is finite
  float f = att_exp(m_run - m_tot);
  float l_tot = l_half * f;
#pragma unroll
  for (int e = 0; e < DB; ++e)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[e][r] *= f;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    f = att_exp(merge_ml[w][0][lane] - m_tot);
    l_tot += merge_ml[w][1][lane] * f;
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[e][r] += merge_o[w * DB * 16 + e * 16 + r][lane] * f;
  }
  l_tot += __shfl_xor(l_tot, 32, 64);
  if (q0 + col < t) {
    float* orow = dst + ((size_t)b * t + qi) * ((size_t)nh * D) + (size_t)head * D;
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        *reinterpret_cast<float4*>(orow + e * 32 + a * 8 + hh * 4) =
            make_float4(o[e][a * 4] / l_tot, o[e][a * 4 + 1] / l_tot, o[e][a * 4 + 2] / l_tot, o[e][a * 4 + 3] / l_tot);
  }
}

// ---- the same with both products as six bf16 terms ------------------------------------------------
// On this chip an f32 MFMA runs on the vector ALU's own datapath: while one executes, no wave of that SIMD issues a
// vector instruction (measured: one wave, v_mfma_f32_32x32x2_f32 + 8 independent v_fma: 113 cycles against 64 + 42 apart;
// with the v_fma in a second wave of the SIMD the same; v_mfma_f32_32x32x16_bf16 + 8 v_fma: 45 against 32 + 42).  The
// kernel above therefore pays for its softmax, masks and staging on top of its 4096 MFMA cycles per block of 32 x 32
// scores, whatever the schedule.  Here the operands are split into three bf16 terms each (x = hi + mid + lo to 2^-25 |x|)
// and a product is the six term pairs whose weight is 2^-16 and up -- (hi, lo), (lo, hi), (mid, mid), (hi, mid),
// (mid, hi), (hi, hi), smallest first, every one accumulated in f32 by v_mfma_f32_32x32x16_bf16: 1536 MFMA cycles per
// block on the matrix cores proper, beside the vector instructions instead of in front of them.  What is dropped is
// 3 x 2^-24 |x| |y| per element, the size of the f32 product's own rounding.
//
// K and V come as planes written by a pass in front (att_planes_kernel), in operand order: per kv head and block of 32
// keys 24 KiB = [K: plane p][k step ks][lane] 16 bytes, then [V: plane p][d block e][key step st][lane] 16 bytes, so
// that an operand is one coalesced 128-bit load straight into the registers the MFMA reads: no LDS in the loop.
//   K operand (p, ks), lane l: K[key = l % 32][16 ks + 8 (l / 32) + 0..7]
//   V operand (p, e, st), lane l: V[key = 16 st + 8 (i / 4) + 4 (l / 32) + i % 4][d = 32 e + l % 32], i = 0..7 -- the keys that
//       registers 8 st .. 8 st + 7 of a lane's score accumulator hold, so the exponentials feed back as the other operand
//       from where they are (as in the kernel above).
// Keys past s are planes of zeros.
typedef __bf16 att_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 att_bf16x2 __attribute__((ext_vector_type(2)));
typedef float att_f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned att_u32x4 __attribute__((ext_vector_type(4)));
constexpr int ATT_PLANE_BLOCK = 1536;  // 16-byte units per block of 32 keys: 2 x 3 planes x 4 operands x 64 lanes

// (x0, x1) -> three words of two bf16 each (x0 in the low half); remainders are exact f32 subtractions.  An infinity or a
// NaN stays whole in the first term (FINITE: the caller knows there is no infinity, e.g. among the exponentials of a softmax;
// a NaN then gives three NaNs).
template <bool FINITE = false>
__device__ __forceinline__ void att_split_pair(float x0, float x1, unsigned& hi, unsigned& mid, unsigned& lo) {
  const unsigned h = __builtin_bit_cast(unsigned, __builtin_convertvector(att_f32x2{x0, x1}, att_bf16x2));
  float r0 = x0 - __uint_as_float(h << 16), r1 = x1 - __uint_as_float(h & 0xffff0000u);
  if (!FINITE) {
    if ((h & 0x7f80u) == 0x7f80u) r0 = 0.f;
    if ((h & 0x7f800000u) == 0x7f800000u) r1 = 0.f;
  }
  const unsigned m = __builtin_bit_cast(unsigned, __builtin_convertvector(att_f32x2{r0, r1}, att_bf16x2));
  const float q0 = r0 - __uint_as_float(m << 16), q1 = r1 - __uint_as_float(m & 0xffff0000u);
  hi = h, mid = m, lo = __builtin_bit_cast(unsigned, __builtin_convertvector(att_f32x2{q0, q1}, att_bf16x2));
}
// eight values -> one operand per plane
template <bool FINITE = false>
__device__ __forceinline__ void att_split8(const float (&x)[8], att_u32x4& hi, att_u32x4& mid, att_u32x4& lo) {
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    unsigned h, md, l;
    att_split_pair<FINITE>(x[2 * m], x[2 * m + 1], h, md, l);
    hi[m] = h, mid[m] = md, lo[m] = l;
  }
}

// k, v: [bh, cap, 64] with rows 0 .. s-1 valid; planes: [bh][ceil(s / 32)][ATT_PLANE_BLOCK] 16-byte units.
// Grid (blocks of 32 keys, bh), 256 threads: thread u writes K operand (ks = u / 64, lane u % 64) and V operand
// (e = u / 128, st = u / 64 % 2, lane u % 64) of all three planes.
__global__ void __launch_bounds__(256) att_planes_kernel(const float* __restrict__ k, const float* __restrict__ v, att_u32x4* __restrict__ planes, int s, size_t cap) {
  const int u = threadIdx.x, l = u & 63, col = l & 31, hh = l >> 5, kb = blockIdx.x;
  const size_t bh = blockIdx.y;
  const float* kbase = k + bh * cap * 64;
  const float* vbase = v + bh * cap * 64;
  att_u32x4* out = planes + (bh * gridDim.x + kb) * ATT_PLANE_BLOCK;
  float x[8];
  att_u32x4 hi, mid, lo;
  {
    const int ks = u >> 6, key = kb * 32 + col;
    if (key < s) {
      const float4 a = *reinterpret_cast<const float4*>(kbase + (size_t)key * 64 + ks * 16 + hh * 8);
      const float4 b = *reinterpret_cast<const float4*>(kbase + (size_t)key * 64 + ks * 16 + hh * 8 + 4);
      x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = 0.f;
    }
    att_split8(x, hi, mid, lo);
    out[(0 * 4 + ks) * 64 + l] = hi;
    out[(1 * 4 + ks) * 64 + l] = mid;
    out[(2 * 4 + ks) * 64 + l] = lo;
  }
  {
    const int e = u >> 7, st = (u >> 6) & 1, d = e * 32 + col;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = kb * 32 + st * 16 + (i >> 2) * 8 + hh * 4 + (i & 3);
      x[i] = key < s ? vbase[(size_t)key * 64 + d] : 0.f;
    }
    att_split8(x, hi, mid, lo);
    att_u32x4* vo = out + 768;
    vo[((0 * 2 + e) * 2 + st) * 64 + l] = hi;
    vo[((1 * 2 + e) * 2 + st) * 64 + l] = mid;
    vo[((2 * 2 + e) * 2 + st) * 64 + l] = lo;
  }
}

__device__ __forceinline__ att_f32x16 att_mma_bf16(const att_u32x4& a, const att_u32x4& b, const att_f32x16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf16x8, a), __builtin_bit_cast(att_bf16x8, b), c, 0, 0, 0);
}

// Same work split, statistics, merge and output as attention_prefill_kernel<64, GROUPS>; q is scaled before it is split
// (scores come out of the MFMAs scaled, and in units of log 2).  planes: what att_planes_kernel wrote for these caches, n_kb blocks per kv head.
// dst_planes != nullptr: the result goes there as the three bf16 planes of rows of nh * 64 elements (what a product of
// these rows on the bf16 matrix pipe reads) and dst is not written.
template <int GROUPS>
__global__ void __launch_bounds__(256 * GROUPS, 2) attention_prefill_x6_kernel(const float* __restrict__ q, const att_u32x4* __restrict__ planes, float* __restrict__ dst,
                                                                               uint16_t* __restrict__ dst_planes, int nh, int nkv, int t, int s, int n_kb, size_t q_row_stride, float scale,
                                                                               const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                               const int* __restrict__ pos, size_t table_len, int interleaved) {
  constexpr int D = 64, H = D / 2, DB = D / 32;
  __shared__ float merge_ml_all[GROUPS][3][2][64];
  __shared__ float merge_o_all[GROUPS][3][DB * 16][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3, group = tid >> 8;
  const int col = lane & 31, hh = lane >> 5;
  const int bh = blockIdx.y, b = bh / nh, head = bh % nh, kvh = head / (nh / nkv);
  const int n_qb = (t + 31) / 32;
  const int qb = GROUPS == 1 ? n_qb - 1 - (int)blockIdx.x : (group == 0 ? n_qb - 1 - (int)blockIdx.x : (int)blockIdx.x);
  const bool idle = GROUPS == 2 && group == 1 && qb == n_qb - 1 - qb;
  float (*merge_ml)[2][64] = merge_ml_all[group];
  float (*merge_o)[64] = merge_o_all[group][0];
  const int q0 = qb * 32;
  const int qi = min(q0 + col, t - 1);
  const int q_pos = s - t + qi;
  const int last_pos = s - t + min(q0 + 31, t - 1);
  const int q_pos_min = s - t + min(q0, t - 1);
  const att_u32x4* pl = planes + ((size_t)b * nkv + kvh) * (size_t)n_kb * ATT_PLANE_BLOCK + lane;
  const int n_blocks = idle ? 0 : last_pos / 32 + 1;

  // K operands of this wave's first block set out before the query row is touched
  att_u32x4 kop[3][4], vop[3][DB][2];
  auto load_k = [&](int kb) {
    const att_u32x4* base = pl + (size_t)min(kb, n_kb - 1) * ATT_PLANE_BLOCK;
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) kop[p][ks] = base[(p * 4 + ks) * 64];
  };
  auto load_v = [&](int kb) {
    const att_u32x4* base = pl + (size_t)min(kb, n_kb - 1) * ATT_PLANE_BLOCK + 768;
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int e = 0; e < DB; ++e)
#pragma unroll
        for (int st = 0; st < 2; ++st) vop[p][e][st] = base[((p * 2 + e) * 2 + st) * 64];
  };
  load_k(wave);

  // this lane's 32 elements of its (rotated, scaled) query row: chunk ks holds columns 16 ks + 8 hh .. + 7.  The scale
  // carries log2(e) as well: scores, running maxima and their differences are in units of log 2, an exponential is one
  // v_exp_f32 (2^x, within an ulp) instead of the seven instructions of att_exp -- this loop is bound by its vector
  // instructions, not by its MFMAs.
  const float scale_log2e = scale * 1.44269504088896340736f;
  att_u32x4 qop[3][4];
  {
    float qr[4][8];
    const float* qrow = q + ((size_t)b * t + qi) * q_row_stride + (size_t)head * D;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const float4 a = *reinterpret_cast<const float4*>(qrow + ks * 16 + hh * 8);
      const float4 c = *reinterpret_cast<const float4*>(qrow + ks * 16 + hh * 8 + 4);
      qr[ks][0] = a.x, qr[ks][1] = a.y, qr[ks][2] = a.z, qr[ks][3] = a.w, qr[ks][4] = c.x, qr[ks][5] = c.y, qr[ks][6] = c.z, qr[ks][7] = c.w;
    }
    if (cos_t) {
      const long long p = (long long)pos[0] + qi;
      const bool ok = p >= 0 && (size_t)(p + 1) * H <= table_len;
      const size_t row = ok ? (size_t)p * H : 0;
      if (interleaved) {
        // pairs (2 i, 2 i + 1) with table entry i: chunk ks holds pairs 8 ks + 4 hh .. + 3
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const float4 c = *reinterpret_cast<const float4*>(cos_t + row + ks * 8 + hh * 4);
          const float4 sn = *reinterpret_cast<const float4*>(sin_t + row + ks * 8 + hh * 4);
          const float cs[4] = {c.x, c.y, c.z, c.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float x1 = qr[ks][2 * i], x2 = qr[ks][2 * i + 1];
            qr[ks][2 * i] = x1 * cs[i] - x2 * ss[i];
            qr[ks][2 * i + 1] = x1 * ss[i] + x2 * cs[i];
          }
        }
      } else {
        // pairs (i, i + 32) with table entry i: chunks ks and ks + 2 hold the two halves of pairs 16 ks + 8 hh .. + 7
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const float4 c0 = *reinterpret_cast<const float4*>(cos_t + row + ks * 16 + hh * 8);
          const float4 c1 = *reinterpret_cast<const float4*>(cos_t + row + ks * 16 + hh * 8 + 4);
          const float4 s0 = *reinterpret_cast<const float4*>(sin_t + row + ks * 16 + hh * 8);
          const float4 s1 = *reinterpret_cast<const float4*>(sin_t + row + ks * 16 + hh * 8 + 4);
          const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w}, ss[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float x1 = qr[ks][i], x2 = qr[ks + 2][i];
            qr[ks][i] = x1 * cs[i] - x2 * ss[i];
            qr[ks + 2][i] = x1 * ss[i] + x2 * cs[i];
          }
        }
      }
      if (!ok) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
          for (int i = 0; i < 8; ++i) qr[ks][i] = NAN;
      }
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int i = 0; i < 8; ++i) qr[ks][i] *= scale_log2e;
      att_split8(qr[ks], qop[0][ks], qop[1][ks], qop[2][ks]);
    }
  }

  float m_run = ATT_MASKED, l_half = 0.f;
  att_f32x16 o[DB];
#pragma unroll
  for (int e = 0; e < DB; ++e)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[e][r] = 0.f;

  // term pairs (plane of the first operand, plane of the second), smallest first
  constexpr int TA[6] = {0, 2, 1, 0, 1, 0}, TB[6] = {2, 0, 1, 1, 0, 0};
  for (int kb = wave; kb < n_blocks; kb += 4) {
    const int key0 = kb * 32;
    load_v(kb);
    att_f32x16 sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
    for (int term = 0; term < 6; ++term)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) sc = att_mma_bf16(kop[TA[term]][ks], qop[TB[term]][ks], sc);
    __builtin_amdgcn_sched_barrier(0);
    load_k(kb + 4);  // into the registers the MFMAs above have read
    float mx = ATT_MASKED;
    if (key0 + 31 > q_pos_min) {  // wave-uniform: only blocks that touch the diagonal have anything to mask
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + (r >> 2) * 8 + hh * 4 + (r & 3);
        sc[r] = key <= q_pos ? sc[r] : ATT_MASKED;
        mx = fmaxf(mx, sc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sc[r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new <= ATT_MASKED ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = __builtin_amdgcn_exp2f(sc[r] - m_use);
      psum += sc[r];
    }
    l_half = l_half * alpha + psum;
    // the exponentials as operands: registers 8 st .. 8 st + 7 are key step st
    att_u32x4 pop[3][2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const float x[8] = {sc[st * 8], sc[st * 8 + 1], sc[st * 8 + 2], sc[st * 8 + 3], sc[st * 8 + 4], sc[st * 8 + 5], sc[st * 8 + 6], sc[st * 8 + 7]};
      att_split8<true>(x, pop[0][st], pop[1][st], pop[2][st]);
    }
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int e = 0; e < DB; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[e][r] *= alpha;
    }
#pragma unroll
    for (int term = 0; term < 6; ++term)
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int e = 0; e < DB; ++e) o[e] = att_mma_bf16(vop[TA[term]][e][st], pop[TB[term]][st], o[e]);
  }

  // merge the four waves' partial results in wave order
  if (wave != 0) {
    merge_ml[wave - 1][0][lane] = m_run;
    merge_ml[wave - 1][1][lane] = l_half;
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int r = 0; r < 16; ++r) merge_o[(wave - 1) * DB * 16 + e * 16 + r][lane] = o[e][r];
  }
  __syncthreads();
  if (wave != 0 || idle) return;
  float m_tot = m_run;
#pragma unroll
  for (int w = 0; w < 3; ++w) m_tot = fmaxf(m_tot, merge_ml[w][0][lane]);
  float f = __builtin_amdgcn_exp2f(m_run - m_tot);
  float l_tot = l_half * f;
#pragma unroll
  for (int e = 0; e < DB; ++e)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[e][r] *= f;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    f = __builtin_amdgcn_exp2f(merge_ml[w][0][lane] - m_tot);
    l_tot += merge_ml[w][1][lane] * f;
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[e][r] += merge_o[w * DB * 16 + e * 16 + r][lane] * f;
  }
  l_tot += __shfl_xor(l_tot, 32, 64);
  if (q0 + col < t) {
    const size_t row = (size_t)b * t + qi, width = (size_t)nh * D;
    float* orow = dst + row * width + (size_t)head * D;
#pragma unroll
    for (int e = 0; e < DB; ++e)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const float y[4] = {o[e][a * 4] / l_tot, o[e][a * 4 + 1] / l_tot, o[e][a * 4 + 2] / l_tot, o[e][a * 4 + 3] / l_tot};
        if (dst_planes) split3_store4(y, dst_planes + row * 3 * width, (size_t)head * D + e * 32 + a * 8 + hh * 4);
        else *reinterpret_cast<float4*>(orow + e * 32 + a * 8 + hh * 4) = make_float4(y[0], y[1], y[2], y[3]);
      }
  }
}

int check_f32(const ughip_slice* s, size_t need, const char* what) {
  if (!s) return set_error(UGHIP_ERR_INVALID, "%s: null slice", what);
  if (s->dtype != UGHIP_F32) return set_error(UGHIP_ERR_INVALID, "%s: unexpected dtype %s, expected F32", what, dtype_name(s->dtype));
  if (s->len < need) return set_error(UGHIP_ERR_BOUNDS, "%s: slice has %zu elements, op needs %zu", what, s->len, need);
  return UGHIP_OK;
}

}  // namespace

extern "C" {

int ughip_causal_softmax_rows(ughip_device* dev, const ughip_slice* src, ughip_slice* dst, size_t bh, size_t s1, size_t s2) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  const size_t n_rows = bh * s1, n = n_rows * s2;
  if (int rc = check_f32(src, n, "causal_softmax src")) return rc;
  if (int rc = check_f32(dst, n, "causal_softmax dst")) return rc;
  if (src == dst) return set_error(UGHIP_ERR_INVALID, "causal_softmax: src and dst alias");
  if (n == 0) return UGHIP_OK;
  if (n_rows > 0x7fffffffull || s2 > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "causal_softmax: shape too large");
  if (int rc = device_activate(dev)) return rc;
  const float* s = static_cast<const float*>(src->ptr);
  float* d = static_cast<float*>(dst->ptr);
  hipStream_t st = dev->stream;
  const int nr = (int)n_rows, nc = (int)s2, is1 = (int)s1;
  const unsigned wave_blocks = (unsigned)((n_rows + 3) / 4);
  if (s2 % 4 == 0 && s2 <= 256) causal_softmax_wave_v4<1><<<wave_blocks, 256, 0, st>>>(s, d, nr, is1, nc);
  else if (s2 % 4 == 0 && s2 <= 512) causal_softmax_wave_v4<2><<<wave_blocks, 256, 0, st>>>(s, d, nr, is1, nc);
  else if (s2 % 4 == 0 && s2 <= 1024) causal_softmax_wave_v4<4><<<wave_blocks, 256, 0, st>>>(s, d, nr, is1, nc);
  else if (s2 % 4 == 0 && s2 <= 2048) causal_softmax_wave_v4<8><<<wave_blocks, 256, 0, st>>>(s, d, nr, is1, nc);
  else causal_softmax_generic<<<nr, 256, 0, st>>>(s, d, is1, nc);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

namespace {
int check_rope_table(const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos, size_t d, const char* what) {
  if (!cos || !sin || cos->dtype != UGHIP_F32 || sin->dtype != UGHIP_F32) return set_error(UGHIP_ERR_INVALID, "%s: cos/sin must be F32 slices", what);
  if (cos->len < d / 2 || sin->len < d / 2) return set_error(UGHIP_ERR_BOUNDS, "%s: rope table shorter than one row of %zu", what, d / 2);
  if (!pos || pos->dtype != UGHIP_I32 || pos->len < 1) return set_error(UGHIP_ERR_INVALID, "%s: pos must be a non-empty I32 slice", what);
  return UGHIP_OK;
}
}  // namespace

int ughip_attention_decode(ughip_device* dev, const ughip_slice* q, const ughip_slice* k, const ughip_slice* v, ughip_slice* dst, size_t b,
                           size_t n_heads, size_t n_kv_heads, size_t s, size_t d, float scale) {
  return ughip_attention_decode_rope(dev, q, k, v, dst, b, n_heads, n_kv_heads, s, d, scale, nullptr, nullptr, nullptr, 0);
}

namespace {
// One query position per head against s keys of caches whose heads are cap rows apart.
// Key ranges per head for `s` keys: one below 800 (the merge launch costs 3 us, what ~700 keys cost one workgroup),
// four up to 1280, then eight -- never more workgroups than CUs (32 heads, measured: 768 keys 8.8 us in one range, 8.9 in
// four; 1024 keys 10.1 / 8.9 / 9.1 in one / four / eight; 2048 keys 15.9 / 10.2 / 9.1).  UGHIP_ATT_SPLIT forces a count
// (tests, tuning).
int decode_ranges(size_t s, size_t heads) {
  const size_t want = s >= 1280 ? 8 : s >= 800 ? 4 : 1;
  int n = (int)std::max<size_t>(1, std::min<size_t>(want, 256 / std::max<size_t>(heads, 1)));
  if (long long v; tune_get(TUNE_ATT_SPLIT, &v)) n = (int)v;
  return std::max(1, std::min(n, 64));
}

// Scratch for the partial rows, grown on demand like the matmul's.
int decode_scratch(ughip_device* dev, size_t bytes, float** out) {
  if (bytes > dev->att_ws_bytes) {
    std::lock_guard<std::mutex> g(dev->mu);
    UGHIP_HIPCHK(hipStreamSynchronize(dev->stream));  // earlier launches may still read the old block
    if (dev->att_ws) (void)hipFree(dev->att_ws);
    dev->att_ws = nullptr;
    dev->att_ws_bytes = 0;
    const size_t want = std::max<size_t>(bytes, (size_t)1 << 20);
    UGHIP_HIPCHK(hipMalloc(&dev->att_ws, want));
    dev->att_ws_bytes = want;
  }
  *out = static_cast<float*>(dev->att_ws);
  return UGHIP_OK;
}

// The launch both entry points share: one workgroup per head and key range, then the merge when a head has several.
int decode_run(ughip_device* dev, size_t heads, const float* q, const float* k, const float* v, float* dst, size_t n_heads, size_t n_kv_heads, size_t s,
               size_t kv_head_stride, size_t q_batch_stride, size_t d, float scale, const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos,
               int interleaved, const float* k_new, const float* v_new, float* k_out, float* v_out) {
  const bool rope = cos != nullptr;
  const int nsplit = decode_ranges(s, heads);
  float* part = nullptr;
  if (nsplit > 1)
    if (int rc = decode_scratch(dev, heads * nsplit * (d + 4) * sizeof(float), &part)) return rc;
  attention_decode_kernel<<<(unsigned)(heads * nsplit), ATT_THREADS, 0, dev->stream>>>(
      q, k, v, dst, (int)n_heads, (int)n_kv_heads, (int)s, kv_head_stride, q_batch_stride, (int)d, scale, rope ? static_cast<const float*>(cos->ptr) : nullptr,
      rope ? static_cast<const float*>(sin->ptr) : nullptr, rope ? static_cast<const int*>(pos->ptr) : nullptr,
      rope ? (cos->len < sin->len ? cos->len : sin->len) : 0, interleaved, k_new, v_new, k_out, v_out, nsplit, part);
  UGHIP_HIPCHK(hipGetLastError());
  if (nsplit > 1) {
    attention_merge_kernel<<<(unsigned)heads, 64, 0, dev->stream>>>(part, dst, nsplit, (int)d);
    UGHIP_HIPCHK(hipGetLastError());
  }
  return UGHIP_OK;
}

int attention_decode_launch(ughip_device* dev, const ughip_slice* q, size_t q_offset, size_t q_row_stride, const ughip_slice* k, const ughip_slice* v,
                            ughip_slice* dst, size_t b, size_t n_heads, size_t n_kv_heads, size_t s, size_t cap, size_t d, float scale, const ughip_slice* cos,
                            const ughip_slice* sin, const ughip_slice* pos, int interleaved) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  const bool rope = cos || sin || pos;
  if (rope)
    if (int rc = check_rope_table(cos, sin, pos, d, "attention_decode")) return rc;
  if (n_kv_heads == 0 || n_heads % n_kv_heads != 0)
    return set_error(UGHIP_ERR_INVALID, "attention_decode: %zu heads are not a multiple of %zu kv heads", n_heads, n_kv_heads);
  if (d < 16 || d > 256 || (d & (d - 1)) != 0) return set_error(UGHIP_ERR_INVALID, "attention_decode: head size %zu is not a power of two in 16..256", d);
  if (s == 0) return set_error(UGHIP_ERR_INVALID, "attention_decode: empty key sequence");
  if (s > cap) return set_error(UGHIP_ERR_INVALID, "attention_decode: %zu keys exceed the cache capacity %zu", s, cap);
  if (s > 0x7fffffffull / 4) return set_error(UGHIP_ERR_INVALID, "attention_decode: too many keys");
  if (q_row_stride == 0) q_row_stride = n_heads * d;
  if (q_row_stride < n_heads * d || (q_offset | q_row_stride) % 4 != 0)
    return set_error(UGHIP_ERR_INVALID, "attention_decode: q offset %zu / row stride %zu do not fit rows of %zu", q_offset, q_row_stride, n_heads * d);
  if (int rc = check_f32(q, b ? q_offset + (b - 1) * q_row_stride + n_heads * d : 0, "attention_decode q")) return rc;
  if (int rc = check_f32(k, b * n_kv_heads * cap * d, "attention_decode k")) return rc;
  if (int rc = check_f32(v, b * n_kv_heads * cap * d, "attention_decode v")) return rc;
  if (int rc = check_f32(dst, b * n_heads * d, "attention_decode dst")) return rc;
  if (dst == q || dst == k || dst == v) return set_error(UGHIP_ERR_INVALID, "attention_decode: dst aliases an input");
  if (b * n_heads == 0) return UGHIP_OK;
  if (b * n_heads > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "attention_decode: too many heads");
  if (int rc = device_activate(dev)) return rc;
  return decode_run(dev, b * n_heads, static_cast<const float*>(q->ptr) + q_offset, static_cast<const float*>(k->ptr), static_cast<const float*>(v->ptr),
                    static_cast<float*>(dst->ptr), n_heads, n_kv_heads, s, cap * d, q_row_stride, d, scale, rope ? cos : nullptr, rope ? sin : nullptr,
                    rope ? pos : nullptr, interleaved, nullptr, nullptr, nullptr, nullptr);
}
}  // namespace

int ughip_attention_step(ughip_device* dev, const ughip_slice* qkv, size_t row_stride, size_t q_offset, size_t k_offset, size_t v_offset, ughip_slice* kcache,
                         ughip_slice* vcache, ughip_slice* dst, size_t b, size_t n_heads, size_t n_kv_heads, size_t s_old, size_t cap, size_t d, float scale,
                         const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos, int interleaved) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  const bool rope = cos || sin || pos;
  if (rope)
    if (int rc = check_rope_table(cos, sin, pos, d, "attention_step")) return rc;
  if (n_kv_heads == 0 || n_heads % n_kv_heads != 0)
    return set_error(UGHIP_ERR_INVALID, "attention_step: %zu heads are not a multiple of %zu kv heads", n_heads, n_kv_heads);
  if (d < 16 || d > 256 || (d & (d - 1)) != 0) return set_error(UGHIP_ERR_INVALID, "attention_step: head size %zu is not a power of two in 16..256", d);
  const size_t s = s_old + 1;
  if (s > cap) return set_error(UGHIP_ERR_BOUNDS, "attention_step: position %zu does not fit a cache of %zu rows", s_old, cap);
  if (s > 0x7fffffffull / 4) return set_error(UGHIP_ERR_INVALID, "attention_step: too many keys");
  const size_t nq = n_heads * d, nk = n_kv_heads * d;
  if (row_stride % 4 != 0 || (q_offset | k_offset | v_offset) % 4 != 0 || q_offset + nq > row_stride || k_offset + nk > row_stride || v_offset + nk > row_stride)
    return set_error(UGHIP_ERR_INVALID, "attention_step: q/k/v at %zu/%zu/%zu do not fit rows of %zu", q_offset, k_offset, v_offset, row_stride);
  if (int rc = check_f32(qkv, b * row_stride, "attention_step qkv")) return rc;
  if (int rc = check_f32(kcache, b * n_kv_heads * cap * d, "attention_step k cache")) return rc;
  if (int rc = check_f32(vcache, b * n_kv_heads * cap * d, "attention_step v cache")) return rc;
  if (int rc = check_f32(dst, b * nq, "attention_step dst")) return rc;
  if (dst == qkv || dst == kcache || dst == vcache || kcache == vcache || qkv == kcache || qkv == vcache)
    return set_error(UGHIP_ERR_INVALID, "attention_step: aliased slices");
  if (b * n_heads == 0) return UGHIP_OK;
  if (b * n_heads > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "attention_step: too many heads");
  if (int rc = device_activate(dev)) return rc;
  const float* base = static_cast<const float*>(qkv->ptr);
  return decode_run(dev, b * n_heads, base + q_offset, static_cast<const float*>(kcache->ptr), static_cast<const float*>(vcache->ptr), static_cast<float*>(dst->ptr),
                    n_heads, n_kv_heads, s, cap * d, row_stride, d, scale, rope ? cos : nullptr, rope ? sin : nullptr, rope ? pos : nullptr, interleaved,
                    base + k_offset, base + v_offset, static_cast<float*>(kcache->ptr), static_cast<float*>(vcache->ptr));
}

int ughip_attention_decode_rope(ughip_device* dev, const ughip_slice* q, const ughip_slice* k, const ughip_slice* v, ughip_slice* dst, size_t b,
                                size_t n_heads, size_t n_kv_heads, size_t s, size_t d, float scale, const ughip_slice* cos, const ughip_slice* sin,
                                const ughip_slice* pos, int interleaved) {
  return attention_decode_launch(dev, q, 0, 0, k, v, dst, b, n_heads, n_kv_heads, s, s, d, scale, cos, sin, pos, interleaved);
}

int ughip_rope_append(ughip_device* dev, const ughip_slice* cache, const ughip_slice* x, ughip_slice* dst, size_t bh, size_t s_old, size_t d,
                      const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos, int interleaved) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (d == 0 || d % 8 != 0) return set_error(UGHIP_ERR_INVALID, "rope_append: head size %zu is not a multiple of 8", d);
  const bool rope = cos || sin || pos;
  if (rope)
    if (int rc = check_rope_table(cos, sin, pos, d, "rope_append")) return rc;
  if (s_old) {
    if (int rc = check_f32(cache, bh * s_old * d, "rope_append cache")) return rc;
  } else if (cache && cache->dtype != UGHIP_F32) {
    return set_error(UGHIP_ERR_INVALID, "rope_append cache: unexpected dtype %s, expected F32", dtype_name(cache->dtype));
  }
  if (int rc = check_f32(x, bh * d, "rope_append x")) return rc;
  if (int rc = check_f32(dst, bh * (s_old + 1) * d, "rope_append dst")) return rc;
  if (dst == cache || dst == x) return set_error(UGHIP_ERR_INVALID, "rope_append: dst aliases an input");
  if (bh == 0) return UGHIP_OK;
  if (s_old + 1 > 0x7fffffffull || d > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "rope_append: shape too large");
  if (int rc = device_activate(dev)) return rc;
  const size_t n4 = bh * (s_old + 1) * d / 4;
  rope_append_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, dev->stream>>>(
      s_old ? static_cast<const float*>(cache->ptr) : nullptr, static_cast<const float*>(x->ptr), static_cast<float*>(dst->ptr), n4, (int)s_old, (int)d,
      rope ? static_cast<const float*>(cos->ptr) : nullptr, rope ? static_cast<const float*>(sin->ptr) : nullptr,
      rope ? static_cast<const int*>(pos->ptr) : nullptr, rope ? (cos->len < sin->len ? cos->len : sin->len) : 0, interleaved);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_kv_append(ughip_device* dev, ughip_slice* cache, const ughip_slice* x, size_t x_offset, size_t x_row_stride, size_t b, size_t n, size_t cap,
                    size_t s_old, size_t t, size_t d, const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos, int interleaved) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (d == 0 || d % 4 != 0) return set_error(UGHIP_ERR_INVALID, "kv_append: head size %zu is not a multiple of 4", d);
  const bool rope = cos || sin || pos;
  if (rope) {
    if (d % 2 != 0) return set_error(UGHIP_ERR_INVALID, "kv_append: odd head size %zu", d);
    if (int rc = check_rope_table(cos, sin, pos, d, "kv_append")) return rc;
  }
  if (s_old + t > cap) return set_error(UGHIP_ERR_BOUNDS, "kv_append: rows %zu..%zu do not fit a cache of %zu rows", s_old, s_old + t, cap);
  if (int rc = check_f32(cache, b * n * cap * d, "kv_append cache")) return rc;
  if (x_row_stride == 0) x_row_stride = n * d;
  if (x_row_stride < n * d || (x_offset | x_row_stride) % 4 != 0)
    return set_error(UGHIP_ERR_INVALID, "kv_append: x offset %zu / row stride %zu do not fit rows of %zu", x_offset, x_row_stride, n * d);
  if (int rc = check_f32(x, b * t ? x_offset + (b * t - 1) * x_row_stride + n * d : 0, "kv_append x")) return rc;
  if (cache == x) return set_error(UGHIP_ERR_INVALID, "kv_append: x aliases the cache");
  const size_t n4 = b * t * n * d / 4;
  if (n4 == 0) return UGHIP_OK;
  if (cap > 0x7fffffffull || t > 0x7fffffffull || n > 0x7fffffffull || d > 0x7fffffffull || n4 > (size_t)0x7fffffff * 256)
    return set_error(UGHIP_ERR_INVALID, "kv_append: shape too large");
  if (int rc = device_activate(dev)) return rc;
  kv_append_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, dev->stream>>>(
      static_cast<float*>(cache->ptr), static_cast<const float*>(x->ptr) + x_offset, x_row_stride, n4, (int)t, (int)n, (int)d, cap, (int)s_old,
      rope ? static_cast<const float*>(cos->ptr) : nullptr, rope ? static_cast<const float*>(sin->ptr) : nullptr,
      rope ? static_cast<const int*>(pos->ptr) : nullptr, rope ? (cos->len < sin->len ? cos->len : sin->len) : 0, interleaved);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_kv_append_pair(ughip_device* dev, ughip_slice* kcache, ughip_slice* vcache, const ughip_slice* x, size_t k_offset, size_t v_offset,
                         size_t x_row_stride, size_t b, size_t n, size_t cap, size_t s_old, size_t t, size_t d, const ughip_slice* cos, const ughip_slice* sin,
                         const ughip_slice* pos, int interleaved) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (d == 0 || d % 4 != 0) return set_error(UGHIP_ERR_INVALID, "kv_append_pair: head size %zu is not a multiple of 4", d);
  const bool rope = cos || sin || pos;
  if (rope) {
    if (d % 2 != 0) return set_error(UGHIP_ERR_INVALID, "kv_append_pair: odd head size %zu", d);
    if (int rc = check_rope_table(cos, sin, pos, d, "kv_append_pair")) return rc;
  }
  if (s_old + t > cap) return set_error(UGHIP_ERR_BOUNDS, "kv_append_pair: rows %zu..%zu do not fit a cache of %zu rows", s_old, s_old + t, cap);
  if (int rc = check_f32(kcache, b * n * cap * d, "kv_append_pair key cache")) return rc;
  if (int rc = check_f32(vcache, b * n * cap * d, "kv_append_pair value cache")) return rc;
  if (x_row_stride == 0 || x_row_stride < n * d || (k_offset | v_offset | x_row_stride) % 4 != 0 || k_offset + n * d > x_row_stride || v_offset + n * d > x_row_stride)
    return set_error(UGHIP_ERR_INVALID, "kv_append_pair: offsets %zu, %zu / row stride %zu do not fit rows of %zu", k_offset, v_offset, x_row_stride, n * d);
  if (int rc = check_f32(x, b * t * x_row_stride, "kv_append_pair x")) return rc;
  if (kcache == x || vcache == x || kcache == vcache) return set_error(UGHIP_ERR_INVALID, "kv_append_pair: the caches and x must be three different slices");
  const size_t n4 = b * t * n * d / 4;
  if (n4 == 0) return UGHIP_OK;
  if (cap > 0x7fffffffull || t > 0x7fffffffull || n > 0x7fffffffull || d > 0x7fffffffull || n4 > (size_t)0x7fffffff * 256)
    return set_error(UGHIP_ERR_INVALID, "kv_append_pair: shape too large");
  if (int rc = device_activate(dev)) return rc;
  kv_append_pair_kernel<<<dim3((unsigned)((n4 + 255) / 256), 2), 256, 0, dev->stream>>>(
      static_cast<float*>(kcache->ptr), static_cast<float*>(vcache->ptr), static_cast<const float*>(x->ptr) + k_offset, static_cast<const float*>(x->ptr) + v_offset,
      x_row_stride, n4, (int)t, (int)n, (int)d, cap, (int)s_old, rope ? static_cast<const float*>(cos->ptr) : nullptr,
      rope ? static_cast<const float*>(sin->ptr) : nullptr, rope ? static_cast<const int*>(pos->ptr) : nullptr,
      rope ? (cos->len < sin->len ? cos->len : sin->len) : 0, interleaved);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

// Several query positions over the caches.  The result goes to `out` [b * t, n_heads * d] as f32, or -- when out_planes is
// given and the kernel that takes these shapes can write them (*wrote_planes says so) -- to out_planes as the three bf16
// planes of those rows.  `out` is checked by the caller (b * t * n_heads * d floats, no alias of an input).
static int attention_prefill_launch(ughip_device* dev, const ughip_slice* q, size_t q_offset, size_t q_row_stride, const ughip_slice* k, const ughip_slice* v, float* out,
                                    uint16_t* out_planes, bool* wrote_planes, size_t b, size_t n_heads, size_t n_kv_heads, size_t t, size_t s, size_t cap, size_t d,
                                    float scale, const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos, int interleaved) {
  if (wrote_planes) *wrote_planes = false;
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  const bool rope = cos || sin || pos;
  if (rope)
    if (int rc = check_rope_table(cos, sin, pos, d, "attention_cached")) return rc;
  if (n_kv_heads == 0 || n_heads % n_kv_heads != 0)
    return set_error(UGHIP_ERR_INVALID, "attention_cached: %zu heads are not a multiple of %zu kv heads", n_heads, n_kv_heads);
  if (d != 32 && d != 64 && d != 128)
    return set_error(UGHIP_ERR_UNSUPPORTED, "attention_cached: head size %zu (32, 64 and 128 are built for more than one query position)", d);
  if (t == 0 || s < t) return set_error(UGHIP_ERR_INVALID, "attention_cached: %zu query positions need at least as many keys, got %zu", t, s);
  if (s > cap) return set_error(UGHIP_ERR_INVALID, "attention_cached: %zu keys exceed the cache capacity %zu", s, cap);
  if (q_row_stride == 0) q_row_stride = n_heads * d;
  if (q_row_stride < n_heads * d || (q_offset | q_row_stride) % 4 != 0)
    return set_error(UGHIP_ERR_INVALID, "attention_cached: q offset %zu / row stride %zu do not fit rows of %zu", q_offset, q_row_stride, n_heads * d);
  if (int rc = check_f32(q, b ? q_offset + (b * t - 1) * q_row_stride + n_heads * d : 0, "attention_cached q")) return rc;
  if (int rc = check_f32(k, b * n_kv_heads * cap * d, "attention_cached k")) return rc;
  if (int rc = check_f32(v, b * n_kv_heads * cap * d, "attention_cached v")) return rc;
  if (b * n_heads == 0) return UGHIP_OK;
  if (b * n_heads > 65535 || s > 0x7fffffffull || cap > 0x7fffffffull) return set_error(UGHIP_ERR_INVALID, "attention_cached: shape too large");
  if (int rc = device_activate(dev)) return rc;
  const unsigned n_qb = (unsigned)((t + 31) / 32);
  const float* cp = rope ? static_cast<const float*>(cos->ptr) : nullptr;
  const float* sp = rope ? static_cast<const float*>(sin->ptr) : nullptr;
  const int* pp = rope ? static_cast<const int*>(pos->ptr) : nullptr;
  const size_t tl = rope ? (cos->len < sin->len ? cos->len : sin->len) : 0;
  const float* qp = static_cast<const float*>(q->ptr) + q_offset;
  const float* kp = static_cast<const float*>(k->ptr);
  const float* vp = static_cast<const float*>(v->ptr);
  float* op = out;
  const int inh = (int)n_heads, inkv = (int)n_kv_heads, it = (int)t, is = (int)s;
  // Two query blocks per workgroup of 8 waves (equal work under the causal mask) once one block per
  // workgroup would give every CU two workgroups anyway; d = 128 needs the whole register file for 4 waves.
  const dim3 paired((n_qb + 1) / 2, (unsigned)(b * n_heads)), single(n_qb, (unsigned)(b * n_heads));
  const bool pair = d <= 64 && (size_t)n_qb * b * n_heads >= 512;
  hipError_t err = hipSuccess;
  auto go = [&](auto kernel, int dd, int groups, dim3 grid) {
    const size_t lds = (size_t)4 * groups * 32 * (2 * dd + 12) * sizeof(float);  // per wave: 32 rows of d + 4 and of d + 8 floats
    err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return;
    kernel<<<grid, 256 * groups, lds, dev->stream>>>(qp, kp, vp, op, inh, inkv, it, is, cap, q_row_stride, scale, cp, sp, pp, tl, interleaved);
  };
  // Head size 64 and enough positions to pay for the pass that writes the planes: both products as six bf16 terms
  // (UGHIP_ATT_X6: 0 never, 1 for any t > 1).
  bool x6 = d == 64 && t >= 256;
  if (long long v; tune_get(TUNE_ATT_X6, &v)) x6 = d == 64 && v != 0;
  if (x6) {
    const size_t n_kb = (s + 31) / 32, bkv = b * n_kv_heads;
    float* ws = nullptr;
    if (int rc = decode_scratch(dev, bkv * n_kb * ATT_PLANE_BLOCK * sizeof(att_u32x4), &ws)) return rc;
    att_u32x4* planes = reinterpret_cast<att_u32x4*>(ws);
    att_planes_kernel<<<dim3((unsigned)n_kb, (unsigned)bkv), 256, 0, dev->stream>>>(kp, vp, planes, is, cap);
    UGHIP_HIPCHK(hipGetLastError());
    if (pair)
      attention_prefill_x6_kernel<2><<<paired, 512, 0, dev->stream>>>(qp, planes, op, out_planes, inh, inkv, it, is, (int)n_kb, q_row_stride, scale, cp, sp, pp, tl, interleaved);
    else
      attention_prefill_x6_kernel<1><<<single, 256, 0, dev->stream>>>(qp, planes, op, out_planes, inh, inkv, it, is, (int)n_kb, q_row_stride, scale, cp, sp, pp, tl, interleaved);
    UGHIP_HIPCHK(hipGetLastError());
    if (wrote_planes) *wrote_planes = out_planes != nullptr;
    return UGHIP_OK;
  }
  if (d == 32 && pair) go(attention_prefill_kernel<32, 2>, 32, 2, paired);
  else if (d == 32) go(attention_prefill_kernel<32, 1>, 32, 1, single);
  else if (d == 64 && pair) go(attention_prefill_kernel<64, 2>, 64, 2, paired);
  else if (d == 64) go(attention_prefill_kernel<64, 1>, 64, 1, single);
  else go(attention_prefill_kernel<128, 1>, 128, 1, single);
  UGHIP_HIPCHK(err);
  UGHIP_HIPCHK(hipGetLastError());
  return UGHIP_OK;
}

int ughip_attention_cached(ughip_device* dev, const ughip_slice* q, size_t q_offset, size_t q_row_stride, const ughip_slice* k, const ughip_slice* v,
                           ughip_slice* dst, size_t b, size_t n_heads, size_t n_kv_heads, size_t t, size_t s, size_t cap, size_t d, float scale,
                           const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos, int interleaved) {
  if (t == 1) return attention_decode_launch(dev, q, q_offset, q_row_stride, k, v, dst, b, n_heads, n_kv_heads, s, cap, d, scale, cos, sin, pos, interleaved);
  if (int rc = check_f32(dst, b * t * n_heads * d, "attention_cached dst")) return rc;
  if (dst == q || dst == k || dst == v) return set_error(UGHIP_ERR_INVALID, "attention_cached: dst aliases an input");
  return attention_prefill_launch(dev, q, q_offset, q_row_stride, k, v, static_cast<float*>(dst->ptr), nullptr, nullptr, b, n_heads, n_kv_heads, t, s, cap, d, scale, cos, sin,
                                  pos, interleaved);
}

int ughip_attention_cached_linear_add_rows(ughip_device* dev, const ughip_slice* q, size_t q_offset, size_t q_row_stride, const ughip_slice* k, const ughip_slice* v,
                                           size_t b, size_t n_heads, size_t n_kv_heads, size_t t, size_t s, size_t cap, size_t d, float scale, const ughip_slice* cos,
                                           const ughip_slice* sin, const ughip_slice* pos, int interleaved, const ughip_slice* w, const ughip_slice* residual,
                                           ughip_slice* dst, size_t n, int product) {
  const char* what = "attention_cached_linear_add_rows";
  if (!dev || !w || !residual || !dst) return set_error(UGHIP_ERR_INVALID, "%s: null argument", what);
  if (t < 2) return set_error(UGHIP_ERR_UNSUPPORTED, "%s: built for several query positions (one position: ughip_attention_step and ughip_gemv_add)", what);
  const size_t m = b * t, width = n_heads * d;
  if (w->dtype != UGHIP_F32 && w->dtype != UGHIP_BF16) return set_error(UGHIP_ERR_INVALID, "%s: the matrix is F32 or BF16, got %s", what, dtype_name(w->dtype));
  if (int rc = check_f32(residual, m * n, "attention_cached_linear_add_rows residual")) return rc;
  if (int rc = check_f32(dst, m * n, "attention_cached_linear_add_rows dst")) return rc;
  if (w->len < n * width) return set_error(UGHIP_ERR_BOUNDS, "%s: the matrix has %zu elements, [%zu, %zu] needs %zu", what, w->len, n, width, n * width);
  if (dst == q || dst == k || dst == v || dst == w) return set_error(UGHIP_ERR_INVALID, "%s: dst aliases an input", what);
  if (m == 0 || width == 0 || n == 0) return UGHIP_OK;
  if (m > 0x7fffffffull || width > 0x7fffffffull / 3) return set_error(UGHIP_ERR_INVALID, "%s: shape too large", what);
  if (int rc = device_activate(dev)) return rc;
  // the rows between the two: f32 (4 bytes an element) or planes (6)
  void* rows = nullptr;
  if (int rc = rows_scratch(dev, m * width * 6, &rows)) return rc;
  const bool want_planes = rows_add_product_reads_planes(dev, w, rows, residual->ptr, dst->ptr, m, n, width, product);
  bool wrote_planes = false;
  if (int rc = attention_prefill_launch(dev, q, q_offset, q_row_stride, k, v, static_cast<float*>(rows), want_planes ? static_cast<uint16_t*>(rows) : nullptr, &wrote_planes, b,
                                        n_heads, n_kv_heads, t, s, cap, d, scale, cos, sin, pos, interleaved))
    return rc;
  return rows_add_product_from(dev, what, static_cast<const float*>(rows), wrote_planes ? static_cast<const uint16_t*>(rows) : nullptr, w,
                               static_cast<const float*>(residual->ptr), static_cast<float*>(dst->ptr), m, n, width, product);
}

}  // extern "C"
