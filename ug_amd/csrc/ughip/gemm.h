// Shared between matmul.hip (dispatch, generic kernels, GEMV) and gemm_tiled.hip (tuned MFMA kernel).
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>

namespace ughip {

struct MMArgs {
  const void* a;
  const void* b;
  void* c;
  int M, N, K;
  long long a_rs, a_cs;  // lhs strides of (m, k), in elements
  long long b_rs, b_cs;  // rhs strides of (k, n), in elements
  long long a_bs, b_bs, c_bs;
  int n_tile = 0;  // set inside the tiled kernel: columns of the workgroup's tile that exist (a last tile may hang over N)
  // [n, k]-major rhs only: b_k_div > 1 -- K tile t of the lhs meets K tile t / b_k_div of the rhs (an lhs whose K tiles come in
  // groups of b_k_div planes of the same columns against one matrix: the rhs tile is fetched once from memory and hit in
  // cache for the other planes); 0 or 1 = tile for tile.  b_kt0 is set inside the tiled kernel: the first K tile of the
  // workgroup's slab.
  int b_k_div = 0, b_kt0 = 0;
};

// Tuned kernel: 256x128, 128x128 or 128x64 tiles, K % 64 == 0 (bf16) / K % 32 == 0 (f32), lhs rows
// contiguous, rhs either [k, n] row-major or [n, k] row-major.  The 128-row tiles take any M, and with
// an [n, k]-major rhs any N: a last tile may hang over the end, it reads the last row again and
// stores only what exists.
// rhs_bf16: the rhs is stored as bf16 under an f32 product ([n, k] row-major only) and widened on its way into LDS.
bool gemm_tiled_supported(int dtype, const MMArgs& p, size_t batch, bool rhs_bf16 = false);
// What the fold of the partial tiles does on its way out (f32 products only).  With an epilogue the product always goes
// through the scratch block, even unsplit, and p.c is the epilogue's output.
struct GemmEpilogue {
  enum Kind { NONE = 0, ADD = 1, SWIGLU = 2 } kind;
  const float* residual;  // ADD: c[m, n] = product + residual[m, n].  SWIGLU: c[m, n / 2] = silu(product[:, :n/2]) * product[:, n/2:]
  bool out_f32 = false;   // a 16-bit product whose fold writes f32 (p.c is then a float buffer)
};
// Bytes of f32 scratch the launch needs (split-K partial tiles for skinny products; 0 for most without an epilogue).
size_t gemm_tiled_workspace_bytes(int dtype, const MMArgs& p, size_t batch, const GemmEpilogue* epi = nullptr);
hipError_t gemm_tiled_launch(hipStream_t stream, int dtype, const MMArgs& p, size_t batch, float* workspace, bool rhs_bf16 = false,
                             const GemmEpilogue* epi = nullptr);
// What the launch above is expected to take (us), from the same per-tile figures that choose its tile and K split; a
// negative value when the kernel does not take the problem.  Used to decide between this kernel and gemm_dma4.
double gemm_tiled_cost_us(int dtype, const MMArgs& p, size_t batch);

// 16-bit types, one wave per SIMD: 256 x 256, 256 x 128 or 128 x 128 tiles (tile codes 256, 128, 64), 4 waves laid out
// 2 x 2 with the accumulators in the accumulation registers, loads that write LDS directly, rhs [n, k]- or [k, n]-major
// (gemm_dma.hip).  Any M, N % 8 == 0, K % 64 == 0 and K >= 256, 16-byte aligned rows, contiguous [batch, M, N] result.
bool gemm_dma_supported(int dtype, const MMArgs& p, size_t batch, int tile);
hipError_t gemm_dma_launch(hipStream_t stream, int dtype, const MMArgs& p, size_t batch, int tile);
// The tile code this kernel should take the problem with, 0 when another kernel should.
int gemm_dma_pick(int dtype, const MMArgs& p, size_t batch);
// The same kernel on three bf16 planes of f32 rows (p.K = 3 k, p.b_k_div = 3, [n, k]-major bf16 matrix), f32 result.
// nsplit == 1: p.c [M, N] is written straight from the accumulators, residual [M, N] added when given.  nsplit > 1 (it
// divides the K tiles, into a multiple of 3 and at least 4 each): workgroups share a tile's K range and leave nsplit
// slabs [M, N] in p.c (scratch), for gemm_fold_f32 to add up.
hipError_t gemm_dma_launch_planes3(hipStream_t stream, const MMArgs& p, int tile, int nsplit, const float* residual, const char* note_tail);
// f32 operands as three bf16 planes each (rows of 3 k elements, the planes of every 64 elements of k side by side; p.K = 6 k):
// the product as six bf16 terms with an f32 result, on either rhs layout.
bool gemm_dma_planes6_supported(const MMArgs& p, size_t batch, int tile);
void gemm_dma_planes6_name(const MMArgs& p, int tile, char* out, size_t out_len);
hipError_t gemm_dma_launch_planes6(hipStream_t stream, const MMArgs& p, size_t batch, int tile);
bool gemm_dma_planes3_split_ok(const MMArgs& p, int nsplit);
// c = fold of nsplit f32 slabs [m, n] in slab order, then the epilogue: NONE, ADD (+ residual[m, n]) or SWIGLU
// (c[m, n / 2] = silu(sum[:, :n / 2]) * sum[:, n / 2:]); n % 8 == 0.
hipError_t gemm_fold_f32(hipStream_t stream, const float* slabs, float* c, size_t m, size_t n, int nsplit, GemmEpilogue::Kind kind, const float* residual);
double gemm_dma_cost_us(const MMArgs& p, size_t batch, int tile);
// The names ughip_last_kernel() reports for the two kernels' launches (tile, split and neighbour folded in): the launches use them, and so
// does ughip_matmul_plan, which answers without launching.
void gemm_dma_name(int dtype, const MMArgs& p, int tile, char* out, size_t out_len);
void gemm_tiled_name(int dtype, const MMArgs& p, size_t batch, bool rhs_bf16, const GemmEpilogue* epi, char* out, size_t out_len);

// f32, one wave per SIMD: 256 x 128 tiles of v_mfma_f32_32x32x2_f32, loads that write LDS directly, rhs [n, k]- or [k, n]-major
// (gemm_dma_f32.hip).  Any M, N % 4 == 0, K % 32 == 0 and K >= 64, 16-byte aligned rows, contiguous [batch, M, N] result.
// _pick: whether this kernel should take the problem ([k, n]-major rhs, whole rounds of 256 tiles or nearly, K >= 512;
// UGHIP_GEMM_SHAPE=8 forces it wherever it applies, any other value keeps it out).
bool gemm_dma_f32_supported(const MMArgs& p, size_t batch);
bool gemm_dma_f32_pick(const MMArgs& p, size_t batch);
hipError_t gemm_dma_f32_launch(hipStream_t stream, const MMArgs& p, size_t batch);
void gemm_dma_f32_name(const MMArgs& p, char* out, size_t out_len);

// 1 .. 128 f32 rows x [m, k] against a bf16 matrix [n, k] as three bf16 terms per row element, the split done inside the product
// (rows_x3.hip): partial sums of `units` consecutive (column tile, k tile) units per workgroup go to f32 slabs in `ws`, a fold adds
// them in a fixed order and applies the epilogue.  n % 8 == 0, k % 64 == 0, 16-byte aligned buffers.
struct RowsX3Plan {
  int units = 0, groups = 0, max_slabs = 0;
  size_t ws_bytes = 0;
};
bool rows_x3_supported(const void* x, const void* w, const void* c, const void* residual, size_t m, size_t n, size_t k);
RowsX3Plan rows_x3_plan(size_t m, size_t n, size_t k, int forced_units, int num_cus);
void rows_x3_name(const RowsX3Plan& pl, GemmEpilogue::Kind kind, char* out, size_t out_len);
hipError_t rows_x3_launch(hipStream_t stream, const float* x, const void* w, float* ws, float* c, size_t m, size_t n, size_t k, const RowsX3Plan& pl, GemmEpilogue::Kind kind,
                          const float* residual);

}  // namespace ughip
