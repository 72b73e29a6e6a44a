// SSA -> HIP lowering for gfx950.  Pure host code: no HIP runtime calls, so it can be
// exercised without a GPU.
#pragma once
#include <stdexcept>
#include <string>
#include <vector>

#include "ughip.h"

namespace ughip {

struct Lowered {
  std::string source;  // complete translation unit handed to hiprtc
  std::string entry;   // extern "C" kernel symbol
  int strategy = UGHIP_STRAT_LITERAL;
  unsigned grid = 1, block = 1, lds_bytes = 0;
  // A grid-wide reduction runs as two kernels, `entry` then `entry2`, that share one device
  // scratch buffer of partial results, passed as a trailing pointer argument to both.
  std::string entry2;
  unsigned grid2 = 0, block2 = 0;
  size_t scratch_part_bytes = 0;
  // Parametric kernels: integer constants of the SSA, passed by value as the last kernel
  // argument (`struct { int v[n]; }`) instead of being printed into the source.
  std::vector<int> kparams;
  std::vector<int> arg_dtype;      // per kernel argument, UGHIP_* dtype
  std::vector<long long> min_len;  // per argument: 1 + largest offset the kernel forms, -1 if unknown
  std::vector<char> arg_written;   // per argument: has a Store
  bool empty_launch = false;       // a loop of the nest has zero trips: nothing to run
};

// Throws std::runtime_error on malformed SSA.  as_written: translate statement by statement for
// the kernel's own launch configuration (a serial loop nest stays one thread's loop nest, what
// ug-cuda/src/code_gen.rs:68-186 emits) instead of re-parallelising it.
Lowered lower_ssa(const ughip_ssa& ssa, const std::string& entry, bool as_written = false);

const char* dtype_c_name(int dtype);
size_t dtype_size(int dtype);

}  // namespace ughip
