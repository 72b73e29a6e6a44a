// f32 GEMM for gfx950 with one multiplying wave per SIMD: 256 x 128 block tile, 4 waves laid out 2 x 2, a wave owns
// 128 x 64 of it as eight 32 x 32 accumulators of v_mfma_f32_32x32x2_f32; a fifth wave sends the loads.  The counterpart
// for f32 of the 16-bit kernel in gemm_dma.hip, replacing the cuBLAS call of ug-cuda/src/gemm.rs:130-332 for large f32
// products with a [k, n]-major rhs (the batched matmul of row-major operands).
//
// Why a second f32 kernel beside the register-staged one (gemm_tiled.hip): on this chip an f32 MFMA executes on the vector
// ALU's datapath -- while one runs, no vector instruction of any wave issues on that SIMD -- and takes 64 cycles, so the
// matrix rate is reached only by a stream of MFMAs with next to nothing vector between them.  Here operand tiles go from
// memory into LDS without passing registers (global_load_lds_dwordx4: no staging loads, stores or address arithmetic in
// the loop), a K tile of 32 is 128 MFMAs per wave (8192 cycles) behind ONE barrier, and the 24-48 LDS reads a multiplying
// wave issues per K tile sit between MFMAs that each leave 60 idle issue cycles.
//
//   LDS, two stages of 48 KiB: A tile [256 rows][32 k] and, rhs [n, k]-major, B tile [128 rows][32 k]: 128-byte rows of 8
//   chunks of 16 bytes, chunk' = chunk ^ ((row / 2) & 7) (the 16 rows a 128-bit operand read names in one pass land on all
//   64 banks).  Rhs [k, n]-major: B tile [32 k][128 n], 512-byte rows of 32 chunks, chunk' = chunk ^ 8 ((k / 4) & 1): the two
//   rows 4 apart that a 32-bit operand read names land in different halves of the banks.  The swizzles are applied to the
//   global address of the lane that fills a position; an instruction fills 1 KiB of LDS in lane order.
//
//   Operands: lane l feeds row / column l % 32 and, of a step of 8 k, k = 4 (l / 32) + j in MFMA j = 0..3 -- four consecutive
//   k per lane are one 128-bit read where k is contiguous ([m, k] lhs, [n, k] rhs) and four 32-bit reads where n is.
//   The operands are swapped (rhs first), so that a lane's accumulator holds four consecutive columns of one result row:
//   16-byte stores, straight from the registers.
//
//   Schedule: one barrier per K tile, between its steps 2 and 3, which says both that tile t + 1 has landed (the loader
//   waits for its loads in front of it) and that nobody reads tile t's stage any more (step 3's operands were read during
//   step 2): behind it the loader sends the DMAs of tile t + 2, which have until the next barrier to land.  Step 3 reads
//   the first operands of tile t + 1.
//
// Any M (rows past the end fetch the last row again and are not stored), N % 4 == 0, K % 32 == 0 and K >= 64, lhs rows
// contiguous and 16-byte aligned, rhs [n, k]- or [k, n]-major with 16-byte aligned rows, contiguous [batch, M, N] result.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>

#include "gemm.h"
#include "internal.h"
#include "ughip.h"

namespace ughip {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 128, BK = 32;
constexpr int A_BYTES = BM * BK * 4, B_BYTES = BN * BK * 4, STAGE_BYTES = A_BYTES + B_BYTES;
constexpr int NDA = A_BYTES / 1024 / 4, NDB = B_BYTES / 1024 / 4, ND = NDA + NDB;  // a quarter of the DMA instructions of a K tile (lhs, rhs, both)

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// Every lane's 16 bytes at base + voff go to LDS at lds_byte_addr + lane * 16.  The compiler does not see the load: the
// waits for it are explicit.
__device__ __forceinline__ void dma16(const void* base, unsigned voff, unsigned lds_byte_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_byte_addr), "v"(voff), "s"(base) : "memory", "m0");
}

// 16-byte unit index of (row, chunk) in a k-contiguous tile of 128-byte rows
__device__ __forceinline__ int kc_idx(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }
// byte offset of (k, n) in the n-contiguous rhs tile
__device__ __forceinline__ int kn_byte(int k, int n) { return k * (BN * 4) + ((((n >> 2) ^ (((k >> 2) & 1) << 3))) << 4) + (n & 3) * 4; }

template <bool B_KN>
__global__ void __launch_bounds__(320) gemm_dma_f32_kernel(MMArgs p, int tiles_m, int tiles_n) {
  extern __shared__ f32x4 lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Block ids go round-robin over the 8 XCDs: id -> (id % 8) * (grid / 8) + id / 8 hands every XCD a contiguous run of
  // tiles (a batch element's tiles, or a block of rows of them), whose operand panels then share that XCD's L2.
  int bid = blockIdx.x;
  if ((gridDim.x & 7) == 0) bid = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
  const int tpb = tiles_m * tiles_n;
  const int batch = bid / tpb;
  const int t_in = bid - batch * tpb;
  const int tm = t_in / tiles_n, tn = t_in - tm * tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;
  const long long lda = p.a_rs, ldb = B_KN ? p.b_rs : p.b_cs;
  const char* Ab = reinterpret_cast<const char*>(static_cast<const float*>(p.a) + (size_t)batch * p.a_bs + (size_t)m0 * lda);
  const char* Bb = reinterpret_cast<const char*>(static_cast<const float*>(p.b) + (size_t)batch * p.b_bs + (B_KN ? (size_t)n0 : (size_t)n0 * ldb));
  const int KT = p.K / BK;
  const int wm = (wave >> 1) * (BM / 2), wn = (wave & 1) * (BN / 2);
  const unsigned lds_addr = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds;
  const int m_last = p.M - 1 - m0, n_left = p.N - n0;

  const long long a_step = BK * 4, b_step = B_KN ? (long long)BK * ldb * 4 : BK * 4;
  if (wave == 4) {
    // The loader: all 48 DMA instructions of a K tile (lhs rows 8 i + lane / 8, then the rhs), none of the MFMAs.  Its
    // instructions are scalar and memory ones: they issue beside the MFMAs of the wave it shares a SIMD with, and the four
    // multiplying waves never wait for the CU's one address unit, which takes 16 cycles per instruction (with every wave
    // sending its twelve behind the barrier each was kept from its MFMAs for 770 cycles per K tile, 8 x 1024^3 134 us;
    // a wave at a time over the tile's steps 131.5; this way 127.9 on the box that gave 129.3 for the latter).
    // Per-lane byte offsets are the same for every K tile (the scalar base moves); rows and chunks past the end of the
    // operand fetch the last one again (their results are not stored).
    unsigned vo[4 * ND];
#pragma unroll
    for (int i = 0; i < 4 * NDA; ++i) {
      const int row = i * 8 + (lane >> 3), cp = lane & 7;
      vo[i] = (unsigned)(min(row, m_last) * lda * 4 + ((cp ^ ((row >> 1) & 7)) << 4));
    }
#pragma unroll
    for (int g = 0; g < 4 * NDB; ++g) {
      if (!B_KN) {
        const int row = g * 8 + (lane >> 3), cp = lane & 7;
        vo[4 * NDA + g] = (unsigned)(min(row, n_left - 1) * ldb * 4 + ((cp ^ ((row >> 1) & 7)) << 4));
      } else {
        const int k = g * 2 + (lane >> 5), cpos = lane & 31;
        const int src = cpos ^ (((k >> 2) & 1) << 3);
        vo[4 * NDA + g] = (unsigned)(k * ldb * 4 + (min(src, n_left / 4 - 1) << 4));
      }
    }
    auto dma_all = [&](int tile) {
      const unsigned st = lds_addr + (tile & 1) * STAGE_BYTES;
#pragma unroll
      for (int i = 0; i < 4 * NDA; ++i) dma16(Ab + tile * a_step, vo[i], st + i * 1024);
#pragma unroll
      for (int g = 0; g < 4 * NDB; ++g) dma16(Bb + tile * b_step, vo[4 * NDA + g], st + A_BYTES + g * 1024);
    };
    dma_all(0);
    if (KT > 1) {
      dma_all(1);
      wait_vmcnt<4 * ND>();
    } else {
      wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_barrier();
    for (int kt = 0; kt + 1 < KT; ++kt) {
      wait_vmcnt<0>();  // tile kt + 1 has landed
      __builtin_amdgcn_s_barrier();
      if (kt + 2 < KT) dma_all(kt + 2);  // into the stage of tile kt, which nobody reads any more
    }
    return;
  }

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // operands of a step of 8 k: fa[set][i]: rows wm + 32 i + lane % 32, fb[set][j]: columns wn + 32 j + lane % 32;
  // element e of either is k = 8 s + 4 (lane / 32) + e
  f32x4 fa[2][4], fb[2][2];
  const int lr = lane & 31, lh = lane >> 5;
  auto read_frags = [&](int stage, int s, int set) {
    const int base = stage * (STAGE_BYTES / 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[set][i] = lds[base + kc_idx(wm + i * 32 + lr, 2 * s + lh)];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (!B_KN) {
        fb[set][j] = lds[base + A_BYTES / 16 + kc_idx(wn + j * 32 + lr, 2 * s + lh)];
      } else {
        const char __attribute__((address_space(3)))* Bs = (const char __attribute__((address_space(3)))*)lds + stage * STAGE_BYTES + A_BYTES;
#pragma unroll
        for (int e = 0; e < 4; ++e) fb[set][j][e] = *(const float __attribute__((address_space(3)))*)(Bs + kn_byte(8 * s + 4 * lh + e, wn + j * 32 + lr));
      }
    }
  };
  auto step = [&](int set) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[set][j][e], fa[set][i][e], acc[i][j], 0, 0, 0);  // rhs first: see above
  };

  // tile 0 has landed (the loader says so); its first operands read
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    read_frags(cur, 1, 1);
    step(0);
    read_frags(cur, 2, 0);
    step(1);
    read_frags(cur, 3, 1);
    step(0);
    if (kt + 1 < KT) {
      wait_lgkmcnt0();  // this wave's last reads of the tile's stage are done
      __builtin_amdgcn_s_barrier();
      read_frags(cur ^ 1, 0, 0);
    }
    step(1);
  }

  // Register r of lane l of accumulator (i, j): result row m0 + wm + 32 i + l % 32, columns n0 + wn + 32 j + 8 (r / 4) + 4 (l / 32) + r % 4.
  // Through the cache: an instruction writes 32 bytes of each of 32 rows, and the four instructions that complete a row's
  // 128-byte line merge there (stored past the cache they reach memory as they are: 8 x 1024^3 157 us against 133).
  float* __restrict__ C = static_cast<float*>(p.c) + (size_t)batch * p.c_bs + (size_t)m0 * p.N + n0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = wm + i * 32 + lr;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = wn + j * 32 + 8 * g + 4 * lh;
        if (row <= m_last && col < n_left) {  // N % 4 == 0: a group of 4 columns exists whole or not at all
          const f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          *reinterpret_cast<f32x4*>(C + (size_t)row * p.N + col) = v;
        }
      }
  }
}

template <bool B_KN>
hipError_t launch(hipStream_t stream, const MMArgs& p, size_t batch) {
  constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static std::atomic<unsigned long long> configured{0};  // one bit per device: the attribute is per device
  auto kernel = gemm_dma_f32_kernel<B_KN>;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
  if (!bit || !(configured.load(std::memory_order_relaxed) & bit)) {
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES)) return e;
    configured.fetch_or(bit, std::memory_order_relaxed);
  }
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const size_t total = batch * (size_t)tiles_m * tiles_n;
  kernel<<<dim3((unsigned)total), dim3(320), LDS_BYTES, stream>>>(p, tiles_m, tiles_n);  // four multiplying waves and the loader
  return hipGetLastError();
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

bool gemm_dma_f32_supported(const MMArgs& p, size_t batch) {
  if (p.M <= 0 || p.N <= 0 || p.N % 4 || p.K % BK || p.K < 2 * BK || batch == 0) return false;
  if (p.a_cs != 1 || p.a_rs % 4 || (batch > 1 && (p.a_bs % 4 || p.b_bs % 4 || p.c_bs % 4))) return false;
  const bool nn = p.b_cs == 1 && p.b_rs != 1, nt = p.b_rs == 1 && p.b_cs != 1;
  if (nn == nt) return false;
  const long long ldb = nn ? p.b_rs : p.b_cs;
  if (ldb % 4) return false;
  // per-lane offsets are 32-bit: the furthest row of a tile has to stay below 4 GiB from the tile's first byte
  if ((unsigned long long)p.a_rs * 4 * BM >= (1ull << 32) || (unsigned long long)ldb * 4 * (nn ? BK : BN) >= (1ull << 32)) return false;
  if (!aligned16(p.a) || !aligned16(p.b) || !aligned16(p.c)) return false;
  return batch * (size_t)((p.M + BM - 1) / BM) * (size_t)((p.N + BN - 1) / BN) < (1u << 24);
}

// Whether this kernel should take the problem: a [k, n]-major rhs (the register-staged kernel transposes such a tile in
// registers on its way to LDS and loses 12 % against its own [n, k]-major form, which in turn is the faster one of the
// two kernels: 8 x 1024^3 142 / 127 us there, 133 / 134 here; 4096^3 1092 / 957 against 1027 / 1011), tiles that fill the
// chip's 256 CUs in whole rounds or nearly (a workgroup holds a CU), and a K long enough for the loop to outweigh the
// tile's way in and out; everything else stays with the register-staged kernel, whose smaller tiles and K split fit
// skinny products.  UGHIP_GEMM_SHAPE=8 forces this kernel wherever it applies, any other value keeps it out.
bool gemm_dma_f32_pick(const MMArgs& p, size_t batch) {
  long long forced = -1;
  if (tune_get(TUNE_GEMM_SHAPE, &forced)) return forced == 8 && gemm_dma_f32_supported(p, batch);
  if (!gemm_dma_f32_supported(p, batch) || p.K < 512 || !(p.b_cs == 1 && p.b_rs != 1)) return false;
  const size_t tiles = batch * (size_t)((p.M + BM - 1) / BM) * (size_t)((p.N + BN - 1) / BN);
  const size_t rounds = (tiles + 255) / 256;
  return tiles >= 224 && (double)tiles >= 0.85 * 256.0 * (double)rounds;
}

void gemm_dma_f32_name(const MMArgs& p, char* out, size_t out_len) {
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  snprintf(out, out_len, "gemm_dma_f32<f32,%s,%dx%d,320t>", nn ? "NN" : "NT", BM, BN);
}

hipError_t gemm_dma_f32_launch(hipStream_t stream, const MMArgs& p, size_t batch) {
  if (!gemm_dma_f32_supported(p, batch)) return hipErrorInvalidValue;
  char name[96];
  gemm_dma_f32_name(p, name, sizeof name);
  note_kernel("%s", name);
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  return nn ? launch<true>(stream, p, batch) : launch<false>(stream, p, batch);
}

}  // namespace ughip
