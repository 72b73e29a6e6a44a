// 16-bit MFMA GEMM for gfx950 with one wave per SIMD: C[b] = A[b] x B[b], f32 accumulate, bf16 or f16.
//
//   block tile BM x BN (256 x 256, 256 x 128 or 128 x 128), K tile 64, 4 waves laid out 2 x 2, each owning BM/2 x BN/2 of the result
//   (any M, N a multiple of 8: a last tile hangs over the end, reads the last row again and stores what exists):
//   (BM / 32) x (BN / 32) accumulators of 16 x 16 (v_mfma_f32_16x16x32: 4 registers each) live in the accumulation
//   registers -- all 256 of them for the largest tile, which a lone wave per SIMD can have -- and leave the
//   architectural registers to two sets of operand fragments; a K tile is two steps of 32: 16 (12, 8) fragment reads
//   feed 64 (32, 16) MFMAs, so the 128 x 128 tile is bound by its LDS reads like the register-staged kernel and is
//   there for products whose larger tiles would leave CUs idle.  The 16 x 16 x 32 shape moves a fifth less through the
//   register file per flop than 32 x 32 x 16 (half the accumulator traffic, twice the operand traffic); under this
//   kernel the chip is held back by power, and the same schedule on the larger shape ran 5-6 % slower.
//   global -> LDS with global_load_lds_dwordx4 (no staging registers), two 64 KiB stages.  The address unit of a CU
//   needs 16 cycles per such instruction and a K tile takes 64 of them, half the tile's time: they are dealt one by one
//   in front of MFMAs over as much of the tile as the stage they fill allows (see the two schedules in the kernel)
//   rhs [n, k]-major: operand fragments are 128-bit LDS reads of k-contiguous rows (XOR-swizzled chunks, conflict free);
//   rhs [k, n]-major: the tile stays [k][n] in LDS (32-byte pieces XOR-swizzled by k so that the reads meet no bank twice)
//   and ds_read_b64_tr_b16 hands every lane 4 consecutive k of its own column: no transposing pass through registers
//   the MFMA operands are swapped (B fragment first): a lane then holds 4 consecutive columns of one result row, the
//   epilogue packs them and goes through LDS so that the result leaves in 16-byte pieces of whole rows
//
// What bounds it: power first, then the address unit.  With U(-1, 1) operands the chip runs this kernel at 1.4-1.8 GHz
// of its 2.4 GHz by box (CU busy cycles against the kernel's duration), and the matrix pipes are busy 80 % of those
// cycles at 8192^3 (89 % with the DMAs taken out, 92 % with the fragment reads taken out as well: the loads cost MFMA
// issue slots, not waiting time -- warming L2 ahead of them or four stages of 32 k instead of two of 64 made it slower).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "gemm.h"
#include "internal.h"
#include "ughip.h"

namespace ughip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

typedef float floatx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ floatx4 mma16(__bf16, const u32x4& a, const u32x4& b, const floatx4& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx4 mma16(_Float16, const u32x4& a, const u32x4& b, const floatx4& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// Every lane's 16 bytes at base + voff go to LDS at lds_byte_addr + lane * 16.  The compiler does not see the load
// (it would wait for all of them before any LDS read): the waits are explicit.
__device__ __forceinline__ void dma16(const void* base, unsigned voff, unsigned lds_byte_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_byte_addr), "v"(voff), "s"(base) : "memory", "m0");
}
// The same in two halves with an MFMA between them as the wait state that the write of M0 needs.  The first half names M0
// as clobbered; nothing can tell the compiler that the second half reads it, so nothing it emits between the two may
// write M0.  This kernel has no instruction that would (no LDS instruction of gfx950 needs M0); the build is held to that
// by a test that reads the compiler's assembly of this file (every global_load_lds is preceded by our own write of M0
// with exactly one MFMA and no other mention of M0 between), and the tests that hold the results bit for bit against the
// register-staged kernel's would show a load gone astray.
__device__ __forceinline__ void dma16_m0(unsigned lds_byte_addr, unsigned stage_offset) {
  asm volatile("s_add_u32 m0, %0, %1" : : "s"(lds_byte_addr), "s"(stage_offset) : "memory", "scc", "m0");
}
__device__ __forceinline__ void dma16_go(const void* base, unsigned voff) { asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base) : "memory"); }

constexpr int BK = 64;

// k-contiguous operand tile ([rows][64] 16-bit): 128-byte rows of 8 chunks, chunk' = chunk ^ ((row / 2) & 7)
__device__ __forceinline__ int kc_idx(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }  // in 16-byte units

// n-contiguous rhs tile ([64 k][BN n] 16-bit): rows of BN / 16 pieces of 32 bytes, piece' = piece ^ h(k) with
// h(k) = (k & 3) | ((k >> 3) & 1) << 2.  A transposing read names, per half wave, 8 rows (k = 8 g + e: e = 0..3 and two values
// of g) and 32 bytes of each; h sends those rows to 8 different pieces, i.e. to all 64 banks once.  (With 64-byte segments
// swizzled by k & 7 the two g of a half wave met in the same banks: 4096^3 95.5 -> 94.2 us on one box.)
__device__ __forceinline__ int kn_h(int k) { return (k & 3) | (((k >> 3) & 1) << 2); }
template <int BN>
__device__ __forceinline__ int kn_byte(int k, int n) {
  return k * (BN * 2) + (((n >> 4) ^ kn_h(k)) << 5) + (n & 15) * 2;
}

// Lane l feeds row / column l % 16, k = 8 (l / 16) .. + 7 of a step of 32.  TWO: the schedule with two barriers per K tile.
// F32OUT: the result leaves as f32 straight from the accumulators (+ residual when given) instead of as T through LDS.
// BDIV > 1 ([n, k]-major rhs): K tile t of the lhs meets K tile t / BDIV of the rhs -- an lhs that holds BDIV planes of every
// 64 columns side by side (a row split into bf16 terms) against one matrix, whose tile then comes from cache for the other planes.
// BDIV == 6 (either rhs layout): both operands hold three planes (hi, mid, lo: planes 0, 1, 2) of every 64 elements of k side
// by side, and K tile t of the loop is term t % 6 of k tile t / 6 of an f32 product taken as six bf16 ones -- (hi, lo),
// (lo, hi), (mid, mid), (hi, mid), (mid, hi), (hi, hi), the small ones first; (mid, lo), (lo, mid) and (lo, lo) stay below
// 2^-24 of the product and are left out.
template <typename T, int BM, int BN, bool B_KN, bool TWO, bool F32OUT = false, int BDIV = 1>
__global__ void __launch_bounds__(256) gemm_dma4(MMArgs p, int tiles_m, int tiles_n, const float* __restrict__ residual) {
  static_assert(BDIV == 1 || BDIV == 6 || !B_KN, "planes of the lhs alone: against an [n, k]-major rhs only");
  extern __shared__ u32x4 lds[];
  constexpr int NI = BM / 32, NJ = BN / 32;            // 16-row and 16-column fragments per wave
  constexpr int NM = NI * NJ;                          // MFMAs per k32 step
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int NDA = BM / 32, NDB = BN / 32, ND = NDA + NDB;  // DMA instructions per wave and K tile
  constexpr int R = NI + NJ;                           // fragment reads per step
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // Block ids go round-robin over the 8 XCDs: id -> (id % 8) * (grid / 8) + id / 8 hands every XCD a contiguous run of
  // tiles, and tiles are numbered in super-rows of 4 tile rows, column by column inside, so that such a run is a 4-row
  // block: its workgroups share few A and B panels in their XCD's L2.
  int bid = blockIdx.x;
  if ((gridDim.x & 7) == 0) bid = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
  const int tpb = tiles_m * tiles_n;
  const int batch = bid / tpb;
  const int t_in = bid - batch * tpb;
  int tm, tn;
  if ((tiles_m & 3) == 0) {
    const int sr = t_in / (4 * tiles_n), rem = t_in - sr * 4 * tiles_n;
    tm = sr * 4 + (rem & 3);
    tn = rem >> 2;
  } else {
    tm = t_in / tiles_n;
    tn = t_in - tm * tiles_n;
  }
  const int m0 = tm * BM, n0 = tn * BN;
  const long long lda = p.a_rs, ldb = B_KN ? p.b_rs : p.b_cs;
  const char* Ab = reinterpret_cast<const char*>(static_cast<const T*>(p.a) + (size_t)batch * p.a_bs + (size_t)m0 * lda);
  const char* Bb = reinterpret_cast<const char*>(static_cast<const T*>(p.b) + (size_t)batch * p.b_bs + (B_KN ? (size_t)n0 : (size_t)n0 * ldb));
  const int KT = p.K / BK;
  const int wm = (wave >> 1) * (BM / 2), wn = (wave & 1) * (BN / 2);
  const unsigned lds_addr = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds;
  // per-lane byte offsets of this wave's DMA instructions (the same for every K tile; the scalar base moves)
  unsigned voff[ND];
  // a last tile may hang over the end of M or N: rows past the end fetch the last row again (their results are not
  // stored), so every address stays inside the operands
  const int m_last = p.M - 1 - m0, n_left = p.N - n0;
#pragma unroll
  for (int i = 0; i < NDA; ++i) {
    const int row = (i * 4 + wave) * 8 + (lane >> 3), cp = lane & 7;
    voff[i] = (unsigned)(min(row, m_last) * lda * 2 + ((cp ^ ((row >> 1) & 7)) << 4));
  }
#pragma unroll
  for (int i = 0; i < NDB; ++i) {
    const int g = i * 4 + wave;
    if (!B_KN) {
      const int row = g * 8 + (lane >> 3), cp = lane & 7;
      voff[NDA + i] = (unsigned)(min(row, n_left - 1) * ldb * 2 + ((cp ^ ((row >> 1) & 7)) << 4));
    } else {
      // one instruction fills 1 KB = 512 / BN rows of k; the lane at LDS position (k, 16-byte chunk cpos) fetches the
      // chunk that the swizzle of the row's 32-byte pieces maps there
      constexpr int CPR = BN / 8;  // 16-byte chunks per row
      const int k = g * (64 / CPR) + lane / CPR, cpos = lane % CPR;
      const int src = (((cpos >> 1) ^ kn_h(k)) << 1) | (cpos & 1);
      voff[NDA + i] = (unsigned)(k * ldb * 2 + (min(src, n_left / 8 - 1) << 4));  // N % 8 == 0: whole 16-byte chunks
    }
  }
  const long long a_step = BK * 2, b_step = B_KN ? (long long)BK * ldb * 2 : BK * 2;
  // which K tile of the lhs and of the rhs in memory the loop's K tile `tile` reads (scalar arithmetic)
  auto a_tile = [&](int tile) -> int {
    if constexpr (BDIV == 6) {
      const int g = tile / 6, r = tile - 6 * g;
      return 3 * g + ((0x010120 >> (4 * r)) & 3);  // planes 0, 2, 1, 0, 1, 0
    } else {
      return tile;
    }
  };
  auto b_tile = [&](int tile) -> int {
    if constexpr (BDIV == 6) {
      const int g = tile / 6, r = tile - 6 * g;
      return 3 * g + ((0x001102 >> (4 * r)) & 3);  // planes 2, 0, 1, 1, 0, 0
    } else {
      return tile / BDIV;
    }
  };
  auto dma = [&](int tile, int idx) {  // idx: compile-time after unrolling
    const unsigned st = lds_addr + (tile & 1) * STAGE_BYTES;
    if (idx < NDA) dma16(Ab + a_tile(tile) * a_step, voff[idx], st + (idx * 4 + wave) * 1024);
    else dma16(Bb + b_tile(tile) * b_step, voff[idx], st + A_BYTES + ((idx - NDA) * 4 + wave) * 1024);
  };
  auto dma_m0 = [&](int tile, int idx) {
    const unsigned in_stage = lds_addr + (idx < NDA ? (idx * 4 + wave) * 1024 : A_BYTES + ((idx - NDA) * 4 + wave) * 1024);  // loop invariant
    dma16_m0(in_stage, (tile & 1) * STAGE_BYTES);
    // the MFMA that follows in the source has to follow in the code: without this the compiler may hoist it above the
    // write of M0, and the load would then come right behind that write, without the wait state it needs
    __builtin_amdgcn_sched_barrier(0);
  };
  auto dma_go = [&](int tile, int idx) {
    if (idx < NDA) dma16_go(Ab + a_tile(tile) * a_step, voff[idx]);
    else dma16_go(Bb + b_tile(tile) * b_step, voff[idx]);
  };

  floatx4 acc[NI][NJ];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  u32x4 fa[2][NI], fb[2][NJ];
  auto read_frag = [&](int stage, int s, int idx, int set) {
    if (idx < NI) {
      fa[set][idx] = lds[stage * (STAGE_BYTES / 16) + kc_idx(wm + idx * 16 + (lane & 15), 4 * s + (lane >> 4))];
    } else if (!B_KN) {
      fb[set][idx - NI] = lds[stage * (STAGE_BYTES / 16) + A_BYTES / 16 + kc_idx(wn + (idx - NI) * 16 + (lane & 15), 4 * s + (lane >> 4))];
    } else {
      // lane q + 4 e of a 16-lane group names row k0 + e, columns 4 q .. 4 q + 3 of the fragment's 16: lane i receives
      // k0 .. k0 + 3 of column i; group g takes k = 8 g .. 8 g + 7 of the step in two such reads
      typedef __attribute__((address_space(3))) s16x4 lds_v4;
      const int g = lane >> 4, li = lane & 15, q = li & 3, e = li >> 2;
      const char __attribute__((address_space(3)))* Bs = (const char __attribute__((address_space(3)))*)lds + stage * STAGE_BYTES + A_BYTES;
      const int n = wn + (idx - NI) * 16 + 4 * q, k0 = s * 32 + 8 * g + e;
      const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4*)(Bs + kn_byte<BN>(k0, n))));
      const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4*)(Bs + kn_byte<BN>(k0 + 4, n))));
      fb[set][idx - NI] = u32x4{lo.x, lo.y, hi.x, hi.y};
    }
  };

  // prologue: tiles 0 and 1 requested, tile 0 landed (tile 1 is waited for at the first barrier that publishes it)
#pragma unroll
  for (int i = 0; i < ND; ++i) dma(0, i);
#pragma unroll
  for (int i = 0; i < ND; ++i) dma(1, i);
  wait_vmcnt<ND>();
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < R; ++i) read_frag(0, 0, i, 0);

  // One barrier per K tile.  Step 0 carries the fragment reads of step 1; step 1 starts behind the barrier that frees
  // this tile's stage and carries the reads of the next tile's step 0 (RN) and all the DMAs of tile kt + 2 (D), which
  // then have a whole step's time to land.  (The memory instructions are pinned one by one in front of MFMAs: a wave
  // alone on its SIMD has nobody to hide a burst of loads behind.)
  auto tile_one = [&](int kt, auto d, auto rn) {
    constexpr bool D = decltype(d)::value, RN = decltype(rn)::value;
    const int cur = kt & 1, nxt = cur ^ 1;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int fc = s, fn = s ^ 1;
      if (s == 1) {
        wait_vmcnt<0>();
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();
      }
      const int n_reads = (s == 0 || RN) ? R : 0, n_dmas = (s == 1 && D) ? ND : 0;
      const int n_ops = n_reads + n_dmas;
#pragma unroll
      for (int g = 0; g < NM; ++g) {
        // the memory instructions in front of MFMA g: those t with t * NM / n_ops == g
        constexpr int PER = (R + ND + NM - 1) / NM;
        static_assert(PER == 1, "at most one memory instruction per MFMA: M0 is written one MFMA ahead of its DMA");
        const int t_lo = (g * n_ops + NM - 1) / NM, t_hi = ((g + 1) * n_ops + NM - 1) / NM;
#pragma unroll
        for (int u = 0; u < PER; ++u) {
          const int t = t_lo + u;
          if (t < t_hi) {
            // reads and DMAs of a step are dealt in proportion: op t is DMA number t * n_dmas / n_ops when that number moves
            const int di = t * n_dmas / n_ops, di_next = (t + 1) * n_dmas / n_ops;
            const bool is_dma = di_next > di;
            const int ri = t - di;
            if (is_dma) dma_m0(kt + 2, di);  // M0 in front of this MFMA, the load behind it: the MFMA is the wait state M0 needs
            else read_frag(s == 0 ? cur : nxt, s == 0 ? 1 : 0, ri, fn);
          }
        }
        const int i = g / NJ, j = g % NJ;
        acc[i][j] = mma16(T(), fb[fc][j], fa[fc][i], acc[i][j]);  // operands swapped: rows of the block are columns of C
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PER; ++u) {
          const int t = t_lo + u;
          if (t < t_hi) {
            const int di = t * n_dmas / n_ops, di_next = (t + 1) * n_dmas / n_ops;
            if (di_next > di) dma_go(kt + 2, di);
          }
        }
      }
    }
  };
  // Two barriers per K tile, so that the DMAs need not all come in one step (64 x 16 cycles of the address unit
  // against the 1024 cycles of a step's MFMAs): 2-3 % faster with an [n, k]-major rhs.  Step 0 reads the fragments of
  // step 1 in front of its first R MFMAs; barrier A, in front of MFMA BAR, then says that nobody reads this tile's
  // stage any more, and the DMAs of tile kt + 2 go out from there to the end of step 1, evenly (EARLY of them in
  // step 0).  Barrier B, at the head of step 1, says that tile kt + 1 has landed (its last DMA went out a whole step
  // ago; the EARLY ones behind it may still be on their way).
  auto tile_two = [&](int kt, auto d, auto rn) {
    constexpr bool D = decltype(d)::value, RN = decltype(rn)::value;
    constexpr int BAR = (R + 4 > NM * 3 / 8 ? R + 4 : NM * 3 / 8) < NM - 1 ? (R + 4 > NM * 3 / 8 ? R + 4 : NM * 3 / 8) : NM - 1;
    constexpr int EARLY = ND * (NM - BAR) / (2 * NM - BAR);
    static_assert(R + ND - EARLY <= NM, "at most one memory instruction per MFMA: M0 is written one MFMA ahead of its DMA");
    const int cur = kt & 1, nxt = cur ^ 1;
#pragma unroll
    for (int g = 0; g < NM; ++g) {
      if (g < R) read_frag(cur, 1, g, 1);
      if (g == BAR) {
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();
      }
      if (D && g > BAR && EARLY > 0) {
        // DMA e goes out in front of the MFMA after this one; M0 is written in front of this one
        const int e = (g - BAR - 1) * EARLY / (NM - BAR - 1), e_next = (g - BAR) * EARLY / (NM - BAR - 1);
        if (e_next > e && e < EARLY) dma_m0(kt + 2, e);
      }
      const int i = g / NJ, j = g % NJ;
      acc[i][j] = mma16(T(), fb[0][j], fa[0][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
      if (D && g > BAR && EARLY > 0) {
        const int e = (g - BAR - 1) * EARLY / (NM - BAR - 1), e_next = (g - BAR) * EARLY / (NM - BAR - 1);
        if (e_next > e && e < EARLY) dma_go(kt + 2, e);
      }
    }
    if (RN) {
      if (D) wait_vmcnt<EARLY>();
      else wait_vmcnt<0>();
      __builtin_amdgcn_s_barrier();
    }
    const int n_reads = RN ? R : 0, n_dmas = D ? ND - EARLY : 0;
    const int n_ops = n_reads + n_dmas;
#pragma unroll
    for (int g = 0; g < NM; ++g) {
      constexpr int PER = (R + ND + NM - 1) / NM;
      const int t_lo = (g * n_ops + NM - 1) / NM, t_hi = ((g + 1) * n_ops + NM - 1) / NM;
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int t = t_lo + u;
        if (t < t_hi) {
          const int di = t * n_dmas / n_ops, di_next = (t + 1) * n_dmas / n_ops;
          if (di_next > di) dma_m0(kt + 2, EARLY + di);
          else read_frag(nxt, 0, t - di, 0);
        }
      }
      const int i = g / NJ, j = g % NJ;
      acc[i][j] = mma16(T(), fb[1][j], fa[1][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int t = t_lo + u;
        if (t < t_hi) {
          const int di = t * n_dmas / n_ops, di_next = (t + 1) * n_dmas / n_ops;
          if (di_next > di) dma_go(kt + 2, EARLY + di);
        }
      }
    }
  };
  auto tile = [&](int kt, auto d, auto rn) {
    if constexpr (TWO) tile_two(kt, d, rn);
    else tile_one(kt, d, rn);
  };
  using Y = std::true_type;
  using N_ = std::false_type;
  for (int kt = 0; kt < KT - 2; ++kt) tile(kt, Y(), Y());
  tile(KT - 2, N_(), Y());
  tile(KT - 1, N_(), N_());

  // Register e of lane l of block (i, j): row wm + 16 i + l % 16, column wn + 16 j + 4 (l / 16) + e.
  if constexpr (F32OUT) {
    // four consecutive f32 per lane: 16-byte stores, 64 contiguous bytes per row and instruction
    float* __restrict__ C = static_cast<float*>(p.c) + (size_t)batch * p.c_bs + (size_t)m0 * p.N + n0;
    const float* __restrict__ Rz = residual ? residual + (size_t)batch * p.c_bs + (size_t)m0 * p.N + n0 : nullptr;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int row = wm + i * 16 + (lane & 15), col = wn + j * 16 + (lane >> 4) * 4;
        if (row <= m_last && col < n_left) {  // N % 8 == 0: a group of 4 columns exists whole or not at all
          floatx4 v = acc[i][j];
          if (Rz) v += *reinterpret_cast<const floatx4*>(Rz + (size_t)row * p.N + col);
          *reinterpret_cast<floatx4*>(C + (size_t)row * p.N + col) = v;
        }
      }
    return;
  }
  // Epilogue through LDS.
  constexpr int PITCH = BN * 2 + 8;
  char __attribute__((address_space(3)))* Cs = (char __attribute__((address_space(3)))*)lds;
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      typedef T tx4 __attribute__((ext_vector_type(4)));
      tx4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (T)acc[i][j][e];
      const int row = wm + i * 16 + (lane & 15), col = wn + j * 16 + (lane >> 4) * 4;
      *(u32x2 __attribute__((address_space(3)))*)(Cs + row * PITCH + col * 2) = __builtin_bit_cast(u32x2, v);
    }
  __syncthreads();
  constexpr int CPR = BN / 8, RPP = 256 / CPR;
  T* __restrict__ C = static_cast<T*>(p.c) + (size_t)batch * p.c_bs + (size_t)m0 * p.N + n0;
  const int c = tid % CPR, r0 = tid / CPR;
#pragma unroll 4
  for (int pass = 0; pass < BM / RPP; ++pass) {
    const int row = pass * RPP + r0;
    const u32x2 lo = *(const u32x2 __attribute__((address_space(3)))*)(Cs + row * PITCH + c * 16);
    const u32x2 hi = *(const u32x2 __attribute__((address_space(3)))*)(Cs + row * PITCH + c * 16 + 8);
    // past the cache: nobody in this launch reads the result, and 256 CUs that store their tiles at the same moment are
    // through sooner when L2 does not hold the lines for the write-back at the kernel's end (8 x 1024^3: 18.7 -> 17.5 us)
    if (row <= m_last && c * 8 < n_left) __builtin_nontemporal_store(u32x4{lo.x, lo.y, hi.x, hi.y}, reinterpret_cast<u32x4*>(C + (size_t)row * p.N + c * 8));
  }
}

template <typename T, int BM, int BN, bool B_KN, bool F32OUT = false, int BDIV = 1>
hipError_t launch(hipStream_t stream, const MMArgs& p, size_t batch, const float* residual = nullptr) {
  constexpr int STAGES = 2 * (BM + BN) * BK * 2, EPI = F32OUT ? 0 : BM * (BN * 2 + 8);
  constexpr int LDS_BYTES = STAGES > EPI ? STAGES : EPI;
  static std::atomic<unsigned long long> configured{0};  // one bit per device: the attribute is per device
  // the schedule with two barriers, except where it does not fit the registers (the transposing reads of the
  // largest tile need pairs of temporaries: 256 registers and spills)
  constexpr bool TWO = !(B_KN && BM == 256 && BN == 256);
  auto kernel = gemm_dma4<T, BM, BN, B_KN, TWO, F32OUT, BDIV>;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
  if (!bit || !(configured.load(std::memory_order_relaxed) & bit)) {
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES)) return e;
    configured.fetch_or(bit, std::memory_order_relaxed);
  }
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const size_t total = batch * (size_t)tiles_m * tiles_n;
  kernel<<<dim3((unsigned)total), dim3(256), LDS_BYTES, stream>>>(p, tiles_m, tiles_n, residual);
  return hipGetLastError();
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

namespace {
// tile codes of the entry points below: 256 = 256 x 256, 128 = 256 x 128, 64 = 128 x 128
bool tile_dims(int tile, int* bm, int* bn) {
  if (tile == 256) *bm = 256, *bn = 256;
  else if (tile == 128) *bm = 256, *bn = 128;
  else if (tile == 64) *bm = 128, *bn = 128;
  else return false;
  return true;
}
}  // namespace

bool gemm_dma_supported(int dtype, const MMArgs& p, size_t batch, int tile) {
  if (dtype != UGHIP_BF16 && dtype != UGHIP_F16) return false;
  int bm, bn;
  if (!tile_dims(tile, &bm, &bn)) return false;
  if (p.M <= 0 || p.N <= 0 || p.N % 8 || p.K % BK || p.K < 4 * BK || batch == 0) return false;
  if (p.a_cs != 1 || p.a_rs % 8 || (batch > 1 && (p.a_bs % 8 || p.b_bs % 8 || p.c_bs % 8))) return false;
  const bool nn = p.b_cs == 1 && p.b_rs != 1, nt = p.b_rs == 1 && p.b_cs != 1;
  if (nn == nt) return false;
  const long long ldb = nn ? p.b_rs : p.b_cs;
  if (ldb % 8) return false;
  // per-lane offsets are 32-bit: the furthest row of a tile has to stay below 4 GiB from the tile's first byte
  if ((unsigned long long)p.a_rs * 2 * bm >= (1ull << 32) || (unsigned long long)ldb * 2 * (nn ? BK : bn) >= (1ull << 32)) return false;
  if (!aligned16(p.a) || !aligned16(p.b) || !aligned16(p.c)) return false;
  return batch * (size_t)((p.M + bm - 1) / bm) * (size_t)((p.N + bn - 1) / bn) < (1u << 24);
}

// Which tile this kernel should take the problem with (a tile code), or 0 when the register-staged kernel is expected to
// be faster.  Both are priced.  This kernel: a fixed cost (launch and first tile, 4 us, and the result's way out at the
// rate of a stream) plus, per round of up to 256 workgroups, the K tiles at a time that grows with the share of the chip
// that is busy -- the chip is power-bound under this kernel, a half-empty round runs at a higher clock: 0.9 + 0.6 x busy
// us per K tile for 256 x 256, 0.62 + 0.2 x busy for 256 x 128, fitted to 4096^3 (108 us), 8 x 1024^3 (20), 3072 x 4096^2
// (92 / 112), 5120^2 x 1024 (54 / 65), 2048 x 2560 x 2048 (40 / 29), 2816^3 (58 / 44), 1280 x 8192 x 2048 (46), 2048^2 x 5632
// (97 / 72).  The other kernel: the model that chooses its own tiles.  Against "256 x 256 tiles when they number 200 or
// more, else 256 x 128 under the same rule" this moves products with 130-250 tiles or a short last round to this kernel
// (3072 x 4096^2: 131 -> 91 us, 5120^2 x 1024: 77 -> 54, 1280 x 8192 x 2048: 64 -> 47, 2048 x 2560 x 2048: 35 -> 29,
// 2304^3: 39 -> 35) and leaves those with about 128 tiles where they were (2048^2 x 5632: 56 us against 72).  The
// 128 x 128 tile (two workgroups per CU) takes what neither fits: 2304^3 35 -> 31 us, 2048 x 2560 x 2048 29 -> 27.
// UGHIP_GEMM_SHAPE=3 / 4 / 5 forces 256 x 256 / 256 x 128 / 128 x 128 where the kernel applies, 0..2 keeps it out (tuning aid).
double gemm_dma_cost_us(const MMArgs& p, size_t batch, int tile) {
  int bm, bn;
  if (!tile_dims(tile, &bm, &bn)) return 1e30;
  const size_t tiles = batch * (size_t)((p.M + bm - 1) / bm) * (size_t)((p.N + bn - 1) / bn);
  const int kt = p.K / BK;
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  double us = 4.0 + (double)batch * p.M * p.N * 2 / 6.4e6;
  // (the figures below were fitted to the kernel on 32 x 32 x 16 MFMAs; on 16 x 16 x 32 and with the loads spread behind two
  // barriers every K tile takes 8 % less: 4096^3 97 us, 8 x 1024^3 18.8, 1024 x 4096^2 41 on 128 x 128 tiles)
  const double layout = (nn ? 1.08 : 1.0) * 0.92;
  if (tile == 64) {
    // two workgroups share a CU: a round is 512 tiles at 0.88 us per K tile; up to 256 tiles run one per CU at
    // 0.47 + 0.16 x busy, the next 256 fill the second slots (2048^3 24.7 us, 2304^3 31.3, 2816^3 45.5, 5120^2 x 1024 61)
    us += kt * 0.88 * (double)(tiles / 512) * layout;
    const size_t left = tiles % 512;
    if (left > 256) us += kt * (0.63 + 0.25 * (double)(left - 256) / 256.0) * layout;
    else if (left) us += kt * (0.47 + 0.16 * (double)left / 256.0) * layout;
    return us;
  }
  const double t0 = tile == 256 ? 0.9 : 0.62, t1 = tile == 256 ? 0.6 : 0.2;
  for (size_t left = tiles; left > 0; left -= left < 256 ? left : 256) {
    const double busy = (left < 256 ? (double)left : 256.0) / 256.0;
    us += kt * (t0 + t1 * busy) * layout;
  }
  return us;
}

int gemm_dma_pick(int dtype, const MMArgs& p, size_t batch) {
  if (long long s; tune_get(TUNE_GEMM_SHAPE, &s)) {
    const int forced = s == 3 ? 256 : s == 4 ? 128 : s == 5 ? 64 : 0;
    return forced && gemm_dma_supported(dtype, p, batch, forced) ? forced : 0;
  }
  int best = 0;
  double best_us = 0;
  for (int tile : {256, 128, 64}) {
    if (!gemm_dma_supported(dtype, p, batch, tile)) continue;
    const double us = gemm_dma_cost_us(p, batch, tile);
    if (!best || us < best_us * 0.97) best = tile, best_us = us;  // the larger tile on a near tie: fewer operand bytes
  }
  if (!best) return 0;
  // the 128 x 128 tile runs at the register-staged kernel's pace (both are bound by their LDS reads): it has to be
  // clearly cheaper to take the product from it
  const double other = gemm_tiled_cost_us(dtype, p, batch);
  return other < 0 || best_us < other * (best == 64 ? 0.95 : 1.0) ? best : 0;
}

void gemm_dma_name(int dtype, const MMArgs& p, int tile, char* out, size_t out_len) {
  int bm = 0, bn = 0;
  tile_dims(tile, &bm, &bn);
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  snprintf(out, out_len, "gemm_dma4<%s,%s,%dx%d,256t>", dtype == UGHIP_F16 ? "f16" : "bf16", nn ? "NN" : "NT", bm, bn);
}

hipError_t gemm_dma_launch(hipStream_t stream, int dtype, const MMArgs& p, size_t batch, int tile) {
  if (!gemm_dma_supported(dtype, p, batch, tile)) return hipErrorInvalidValue;
  int bm = 0, bn = 0;
  tile_dims(tile, &bm, &bn);
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  {
    char name[96];
    gemm_dma_name(dtype, p, tile, name, sizeof name);
    note_kernel("%s", name);
  }
#define UGHIP_DMA_CASE(T)                                                                                                  \
  if (tile == 256) return nn ? launch<T, 256, 256, true>(stream, p, batch) : launch<T, 256, 256, false>(stream, p, batch); \
  if (tile == 128) return nn ? launch<T, 256, 128, true>(stream, p, batch) : launch<T, 256, 128, false>(stream, p, batch); \
  return nn ? launch<T, 128, 128, true>(stream, p, batch) : launch<T, 128, 128, false>(stream, p, batch);
  if (dtype == UGHIP_F16) {
    UGHIP_DMA_CASE(_Float16)
  }
  UGHIP_DMA_CASE(__bf16)
#undef UGHIP_DMA_CASE
}

// bf16 planes of f32 rows (three per 64 columns: p.K = 3 k, p.b_k_div = 3) against an [n, k]-major bf16 matrix, f32 result
// [M, N] (+ residual [M, N] when given), or nsplit slabs of it: the splits of K run as the kernel's batches, with the
// batch strides of the operands standing for a split's offset in K (a whole number of groups of three planes).
bool gemm_dma_planes3_split_ok(const MMArgs& p, int nsplit) {
  if (nsplit < 1 || p.K % (BK * nsplit)) return false;
  const int kts = p.K / BK / nsplit;
  return kts % 3 == 0 && kts >= 4;
}

hipError_t gemm_dma_launch_planes3(hipStream_t stream, const MMArgs& p, int tile, int nsplit, const float* residual, const char* note_tail) {
  if (p.b_k_div != 3 || !(p.b_rs == 1 && p.b_cs != 1) || !gemm_dma_planes3_split_ok(p, nsplit) || (nsplit > 1 && residual)) return hipErrorInvalidValue;
  MMArgs q = p;
  if (nsplit > 1) {
    q.K = p.K / nsplit;
    q.a_bs = q.K, q.b_bs = q.K / 3, q.c_bs = (long long)p.M * p.N;
  }
  if (!gemm_dma_supported(UGHIP_BF16, q, (size_t)nsplit, tile)) return hipErrorInvalidValue;
  if (residual && !aligned16(residual)) return hipErrorInvalidValue;
  int bm = 0, bn = 0;
  tile_dims(tile, &bm, &bn);
  char split[24] = "";
  if (nsplit > 1) snprintf(split, sizeof split, ",splitK=%d", nsplit);
  note_kernel("gemm_dma4<bf16,NT,%dx%d,256t,3 planes%s,f32 out%s>", bm, bn, split, note_tail ? note_tail : "");
  if (tile == 256) return launch<__bf16, 256, 256, false, true, 3>(stream, q, (size_t)nsplit, residual);
  if (tile == 128) return launch<__bf16, 256, 128, false, true, 3>(stream, q, (size_t)nsplit, residual);
  return launch<__bf16, 128, 128, false, true, 3>(stream, q, (size_t)nsplit, residual);
}


// Both operands as three bf16 planes per 64 elements of k (p.K = 6 k, rows of 3 k elements), f32 result: see BDIV == 6.
bool gemm_dma_planes6_supported(const MMArgs& p, size_t batch, int tile) { return p.K % (6 * BK) == 0 && gemm_dma_supported(UGHIP_BF16, p, batch, tile); }

void gemm_dma_planes6_name(const MMArgs& p, int tile, char* out, size_t out_len) {
  int bm = 0, bn = 0;
  tile_dims(tile, &bm, &bn);
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  snprintf(out, out_len, "gemm_dma4<bf16,%s,%dx%d,256t,6 terms of 3 x 3 planes,f32 out>", nn ? "NN" : "NT", bm, bn);
}

hipError_t gemm_dma_launch_planes6(hipStream_t stream, const MMArgs& p, size_t batch, int tile) {
  if (!gemm_dma_planes6_supported(p, batch, tile)) return hipErrorInvalidValue;
  char name[112];
  gemm_dma_planes6_name(p, tile, name, sizeof name);
  note_kernel("%s", name);
  const bool nn = p.b_cs == 1 && p.b_rs != 1;
  if (tile == 256) return nn ? launch<__bf16, 256, 256, true, true, 6>(stream, p, batch) : launch<__bf16, 256, 256, false, true, 6>(stream, p, batch);
  if (tile == 128) return nn ? launch<__bf16, 256, 128, true, true, 6>(stream, p, batch) : launch<__bf16, 256, 128, false, true, 6>(stream, p, batch);
  return nn ? launch<__bf16, 128, 128, true, true, 6>(stream, p, batch) : launch<__bf16, 128, 128, false, true, 6>(stream, p, batch);
}

}  // namespace ughip
