// Shared between the translation units of libughip.so; not part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <map>
#include <mutex>
#include <vector>
#include <unordered_map>
#include <string>

#include "ughip.h"

struct CachedModule {
  hipModule_t module = nullptr;
  hipFunction_t function = nullptr, function2 = nullptr;
};

struct ughip_device {
  std::atomic<int> refs{1};
  int ordinal = 0;
  hipStream_t stream = nullptr;
  std::string arch;
  int num_cus = 0;
  std::mutex mu;
  // Size-class free lists: freed blocks are reused by later allocations on the same stream.
  std::unordered_map<size_t, std::vector<void*>> pool;  // free blocks by size class
  size_t pool_bytes = 0, live_bytes = 0;
  bool zero_fill = true;
  std::map<std::string, CachedModule> modules;  // generated source -> loaded code object
  // Scratch of the split-K matmul (partial tiles); grown on demand, reused by every launch of the
  // device's one stream, freed with the device.
  void* gemm_ws = nullptr;
  size_t gemm_ws_bytes = 0;
  // This device's address of the static array behind ughip_matmul_noalloc (hipGetSymbolAddress at device creation).
  void* static_scratch = nullptr;
  // Partial rows of single-query attention over a long cache (one per head and key range); same life cycle.
  void* att_ws = nullptr;
  size_t att_ws_bytes = 0;
  // What lies between the launches of one call on rows (ughip_rms_linear_rows, ughip_rms_mlp_rows); same life cycle.
  void* rows_ws = nullptr;
  size_t rows_ws_bytes = 0;
};

struct ughip_slice {
  ughip_device* dev = nullptr;
  void* ptr = nullptr;
  int dtype = UGHIP_F32;
  size_t len = 0, cap_bytes = 0;
};

namespace ughip {

// Records the thread-local message returned by ughip_last_error() and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Records what ughip_last_kernel() returns: the hand-written kernel the calling thread launched last.
void note_kernel(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int device_activate(ughip_device* d);
int matmul_scratch_setup(ughip_device* dev);  // matmul.hip
// For entry points of other files that end in a projection with its residual (matmul.hip): the device's block for what lies
// between their launches, grown to `bytes`; whether dst[m, n] = x w^T + residual would read x as three bf16 planes from
// memory; and that product on f32 rows x, or on `planes` when they were written already (x is then only a stand-in).
int rows_scratch(ughip_device* dev, size_t bytes, void** out);
bool rows_add_product_reads_planes(ughip_device* dev, const ughip_slice* w, const void* x, const void* residual, const void* dst, size_t m, size_t n, size_t k, int product);
int rows_add_product_from(ughip_device* dev, const char* what, const float* x, const uint16_t* planes, const ughip_slice* w, const float* residual, float* dst, size_t m,
                          size_t n, size_t k, int product);
const char* dtype_name(int dt);

// Tuning switches (tile / split / kernel-family overrides for measurements and tests).  The table is filled once per
// process from the environment (UGHIP_<NAME>), the first time any switch is asked for, and changes afterwards only
// through ughip_set_tuning: dispatch reads an atomic, never the environment, so a launch thread and a test that
// flips a switch do not meet in getenv / setenv.
enum TuneKey {
  TUNE_GEMM_SHAPE,          // 0..2: a gemm_tiled tile (keeps gemm_dma4 out); 3 / 4 / 5: gemm_dma4 with 256x256 / 256x128 / 128x128; 8: gemm_dma_f32 for f32 products
  TUNE_GEMM_SPLIT,          // K split of gemm_tiled
  TUNE_GEMM_4WAVES,         // (set at all) the 256-thread form of the 256x128 tile
  TUNE_GEMV_KS,             // waves per output column of the GEMV family: 1, 2 or 4
  TUNE_GEMV_ROWS,           // rows per workgroup of fused_gemv_bf16_rows: 1, 2, 4 or 8
  TUNE_GEMV_BF16_ROWS,      // 0: bf16 matrices take the f32 kernels' lane layout
  TUNE_X3_DMA,              // three-term bf16 products: 0 keeps gemm_tiled, 3 / 4 / 5 force a gemm_dma4 tile
  TUNE_X3_SPLIT,            // K split of the three-term product on gemm_dma4
  TUNE_X3_ROWS,             // three-term bf16 products of 65 .. 128 rows: 0 keeps the kernels that take planes, n > 0 forces n units per workgroup of rows_x3
  TUNE_ATT_SPLIT,           // key ranges per head of single-query attention
  TUNE_NO_PARAMETRIC,       // (set at all) shapes stay literals in generated kernels
  TUNE_NO_NT_LOADS,         // (set at all) the grid-wide reduction reads with ordinary loads
  TUNE_GRID_REDUCE_BLOCKS,  // workgroups of the grid-wide reduction's first stage
  TUNE_GRID_REDUCE_THREADS, // threads per workgroup there: 64, 128, 256, 512 or 1024
  TUNE_NO_NT_STORES,        // (set at all) generated elementwise kernels store through the cache
  TUNE_SOFTMAX_STREAM,      // ughip_softmax_rows: 0 never takes the resident wave-per-row kernel, n > 0 forces it onto n workgroups
  TUNE_ATT_X6,              // attention over several query positions, head size 64: 0 keeps the f32 products, 1 takes six bf16 terms for any count
  TUNE_MATMUL_X6,           // f32 products of ughip_matmul: 1 takes those of contiguous operands with k % 64 == 0, n % 8 == 0 as six bf16 terms on the bf16 matrix pipe
  TUNE_COUNT
};
bool tune_get(TuneKey k, long long* value);  // false: the switch is not set
inline bool tune_on(TuneKey k) {
  long long v;
  return tune_get(k, &v);
}

}  // namespace ughip

#define UGHIP_HIPCHK(expr)                                                                                 \
  do {                                                                                                     \
    hipError_t e_ = (expr);                                                                                \
    if (e_ != hipSuccess) return ughip::set_error(UGHIP_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)
