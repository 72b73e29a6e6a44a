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
const char* dtype_name(int dt);

}  // namespace ughip

#define UGHIP_HIPCHK(expr)                                                                                 \
  do {                                                                                                     \
    hipError_t e_ = (expr);                                                                                \
    if (e_ != hipSuccess) return ughip::set_error(UGHIP_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)
