// SSA -> HIP lowering for gfx950 (CDNA4, wave64).
//
// The input is ug's flat `ssa::Kernel` (ug-core/src/lang.rs:690-753).  Two routes:
//
//  * kernels that already speak GPU (Special / Barrier / ReduceLocal / DefineLocal / If,
//    e.g. ug-core/src/samples.rs:52-228) are translated statement by statement and
//    launched with the SSA's own LaunchConfig, like ug-cuda/src/code_gen.rs:68-186 does;
//
//  * serial loop nests -- what `op::Kernel::lower(&Opts::default())` produces for a device
//    whose `use_grid()` is false (ug-core/src/lower_op.rs:409-491, schedule.rs:162-188) --
//    are re-parallelised here.  The nest is recovered from the flat list, every value gets
//    the set of loops it depends on, reductions (`DefineAcc / Range / fold / Assign /
//    EndRange`, lower_op.rs:365-391) that do not depend on an enclosing loop are computed
//    once per "row" instead of once per element, and the work is mapped on the machine:
//      ELEMENTWISE  flat thread per 4 consecutive elements;
//      ROW_BLOCK    one workgroup (or one wave64) per row, DPP + LDS reduction;
//      ROW_THREAD   one thread per row when the reduced dim is the strided one;
//      GRID_REDUCE  many workgroups per row, partials + "last block finishes" second stage
//                   in a fixed order (deterministic).
//    Anything the analysis cannot prove safe falls back to a literal single-thread kernel
//    with the exact serial semantics of the CPU backend (cpu_code_gen.rs:68-186).
#include "lower_hip.h"

#include "internal.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <sstream>

namespace ughip {

const char* dtype_c_name(int dtype) {
  switch (dtype) {
    case UGHIP_BF16: return "__bf16";
    case UGHIP_F16: return "_Float16";
    case UGHIP_F32: return "float";
    case UGHIP_I32: return "int";
    case UGHIP_I64: return "long long";
  }
  throw std::runtime_error("unknown dtype " + std::to_string(dtype));
}

size_t dtype_size(int dtype) {
  switch (dtype) {
    case UGHIP_BF16:
    case UGHIP_F16: return 2;
    case UGHIP_F32:
    case UGHIP_I32: return 4;
    case UGHIP_I64: return 8;
  }
  throw std::runtime_error("unknown dtype " + std::to_string(dtype));
}

namespace {

using i64 = long long;

[[noreturn]] void fail(const std::string& m) { throw std::runtime_error("ssa lowering: " + m); }

bool is_float(int dt) { return dt == UGHIP_F32 || dt == UGHIP_F16 || dt == UGHIP_BF16; }

// ---------------------------------------------------------------------------------------
// Device-side helpers prepended to every generated translation unit.
const char* kPrelude = R"HIP(
#define UG_DEV static __device__ inline __attribute__((always_inline))
UG_DEV int ug_lane() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }
template <int CTRL> UG_DEV int ug_dpp_i(int v) { return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false); }
UG_DEV int ug_bperm_i(int v, int src_lane) { return __builtin_amdgcn_ds_bpermute(src_lane << 2, v); }
template <typename T> struct ug_x;
template <> struct ug_x<int> {
  template <int C> UG_DEV int dpp(int v) { return ug_dpp_i<C>(v); }
  UG_DEV int bperm(int v, int l) { return ug_bperm_i(v, l); }
};
template <> struct ug_x<float> {
  template <int C> UG_DEV float dpp(float v) { return __builtin_bit_cast(float, ug_dpp_i<C>(__builtin_bit_cast(int, v))); }
  UG_DEV float bperm(float v, int l) { return __builtin_bit_cast(float, ug_bperm_i(__builtin_bit_cast(int, v), l)); }
};
template <> struct ug_x<long long> {
  template <int C> UG_DEV long long dpp(long long v) {
    unsigned lo = (unsigned)v, hi = (unsigned)((unsigned long long)v >> 32);
    lo = (unsigned)ug_dpp_i<C>((int)lo); hi = (unsigned)ug_dpp_i<C>((int)hi);
    return (long long)(((unsigned long long)hi << 32) | lo);
  }
  UG_DEV long long bperm(long long v, int l) {
    unsigned lo = (unsigned)v, hi = (unsigned)((unsigned long long)v >> 32);
    lo = (unsigned)ug_bperm_i((int)lo, l); hi = (unsigned)ug_bperm_i((int)hi, l);
    return (long long)(((unsigned long long)hi << 32) | lo);
  }
};
struct ug_sum { template <typename T> UG_DEV T f(T a, T b) { return a + b; } };
struct ug_max {
  UG_DEV float f(float a, float b) { return fmaxf(a, b); }
  UG_DEV int f(int a, int b) { return a > b ? a : b; }
  UG_DEV long long f(long long a, long long b) { return a > b ? a : b; }
};
struct ug_min {
  UG_DEV float f(float a, float b) { return fminf(a, b); }
  UG_DEV int f(int a, int b) { return a < b ? a : b; }
  UG_DEV long long f(long long a, long long b) { return a < b ? a : b; }
};
// Butterfly over the 64 lanes of a wave: quad_perm xor1, xor2, row_half_mirror, row_mirror
// on the DPP path, then two bpermutes across the 16-lane rows.  Needs all 64 lanes active.
// Every lane returns the same bits (each step combines two values symmetrically).
template <typename Op, typename T> UG_DEV T ug_wave_reduce(T v) {
  v = Op::f(v, ug_x<T>::template dpp<0xB1>(v));
  v = Op::f(v, ug_x<T>::template dpp<0x4E>(v));
  v = Op::f(v, ug_x<T>::template dpp<0x141>(v));
  v = Op::f(v, ug_x<T>::template dpp<0x140>(v));
  const int lane = ug_lane();
  v = Op::f(v, ug_x<T>::bperm(v, lane ^ 16));
  v = Op::f(v, ug_x<T>::bperm(v, lane ^ 32));
  return v;
}
// Reduction over a workgroup of NW full waves; every thread returns the total.
template <typename Op, typename T, int NW> UG_DEV T ug_block_reduce(T v) {
  v = ug_wave_reduce<Op, T>(v);
  if (NW == 1) return v;
  __shared__ T s[NW > 1 ? NW : 1];
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = v;
  __syncthreads();
  T r = s[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = Op::f(r, s[i]);
  return r;
}
// ReduceLocal for kernels that bring their own launch shape: any blockDim.x <= 1024.
template <typename Op, typename T> UG_DEV T ug_block_reduce_dyn(T v) {
  __shared__ T s[1024];
  const int n = blockDim.x, t = threadIdx.x;
  __syncthreads();
  if ((n & 63) == 0) {
    v = ug_wave_reduce<Op, T>(v);
    if ((t & 63) == 0) s[t >> 6] = v;
    __syncthreads();
    T r = s[0];
    for (int i = 1; i < (n >> 6); ++i) r = Op::f(r, s[i]);
    return r;
  }
  s[t] = v;
  __syncthreads();
  int p = 1;
  while (p < n) p <<= 1;
  for (int st = p >> 1; st > 0; st >>= 1) {
    if (t < st && t + st < n) s[t] = Op::f(s[t], s[t + st]);
    __syncthreads();
  }
  return s[0];
}
)HIP";

// ---------------------------------------------------------------------------------------
struct VType {
  bool valid = false, ptr = false, local = false;
  int dtype = UGHIP_F32;
};

struct LoopInfo {
  int begin = 0, end = 0, parent = -1, depth = 0;
  bool cb = false;  // constant bounds
  i64 lo = 0, up = 0, step = 1, trip = 0;
};

struct Itv {
  bool known = false;
  i64 lo = 0, hi = 0;
};

struct Aff {
  bool ok = false;
  i64 c = 0;
  std::map<int, i64> t;  // loop id -> coefficient
};

struct Region {
  int range = 0, end = 0, acc = 0, fold = 0, assign = 0, op = 0, loop = 0;
  bool acc_is_lhs = true;
  i64 trip = 0;
};

struct Item {
  int kind = 0;  // 0 instr, 1 parallel-reduce region, 2 verbatim loop
  int idx = 0, end = 0, region = -1;
  uint64_t deps = 0;
};

class Lowering {
 public:
  Lowering(const ughip_ssa& s, const std::string& entry, bool as_written) : s_(s), I_(s.instrs), n_((int)s.n_instrs), entry_(entry), as_written_(as_written) {}

  Lowered run() {
    validate();
    out_.entry = entry_;
    out_.arg_dtype.resize(s_.n_args);
    out_.min_len.assign(s_.n_args, 0);
    out_.arg_written.assign(s_.n_args, 0);
    for (size_t a = 0; a < s_.n_args; ++a) out_.arg_dtype[a] = s_.args[a].dtype;
    bool gpu_style = false;
    for (int i = 0; i < n_; ++i) {
      switch (I_[i].op) {
        case UGHIP_I_SPECIAL:
        case UGHIP_I_DEFINE_LOCAL:
        case UGHIP_I_BARRIER:
        case UGHIP_I_REDUCE_LOCAL:
        case UGHIP_I_IF:
        case UGHIP_I_END_IF: gpu_style = true; break;
        default: break;
      }
    }
    compute_intervals(gpu_style);
    compute_bounds();
    if (out_.empty_launch) {
      emit_literal(1, 1);  // valid source, never launched
      return out_;
    }
    if (gpu_style || as_written_) {
      emit_literal(s_.grid_dim ? s_.grid_dim : 1, s_.block_dim ? s_.block_dim : 1);
      return out_;
    }
    compute_deps();
    compute_affine();
    if (!plan_auto()) emit_literal(1, 1);
    return out_;
  }

 private:
  const ughip_ssa& s_;
  const ughip_instr* I_;
  int n_;
  std::string entry_;
  bool as_written_ = false;
  mutable bool nt_loads_ = false;  // loads of the region being emitted bypass cache allocation
  bool nt_stores_ = false;         // stores to kernel arguments go past the cache (set while an elementwise kernel is emitted)
  Lowered out_;

  std::vector<VType> vt_;
  std::vector<LoopInfo> loops_;
  std::vector<int> loop_id_;   // per instr: loop id if Range, else -1
  std::vector<int> encl_;      // per instr: innermost enclosing loop id (Range belongs to its parent)
  std::vector<int> arg_of_;    // per instr: kernel-arg index if DefineGlobal
  std::vector<bool> guarded_;  // per instr: inside an If
  std::vector<int> if_of_;     // per instr: innermost enclosing If (instr index), -1 if none; for an If, the one around it
  std::vector<uint64_t> dep_;  // per var: loops it depends on
  std::vector<Itv> itv_;
  std::vector<Aff> aff_;

  // ---- helpers ------------------------------------------------------------------------
  bool const_int(const ughip_a& a, i64* v) const {
    if (a.is_const) {
      if (a.dtype == UGHIP_I32 || a.dtype == UGHIP_I64) {
        *v = a.i;
        return true;
      }
      return false;
    }
    const ughip_instr& d = I_[a.var];
    if (d.op == UGHIP_I_CONST && d.a.is_const && (d.a.dtype == UGHIP_I32 || d.a.dtype == UGHIP_I64)) {
      *v = d.a.i;
      return true;
    }
    return false;
  }

  void check_a(const ughip_a& a, int at) const {
    if (a.is_const) {
      if (a.dtype > UGHIP_I64) fail("bad const dtype at " + std::to_string(at));
      return;
    }
    if ((int)a.var >= n_) fail("operand var out of range at " + std::to_string(at));
    if ((int)a.var >= at) fail("operand var used before definition at " + std::to_string(at));
  }

  void validate() {
    if (n_ <= 0) fail("empty kernel");
    vt_.assign(n_, VType());
    loop_id_.assign(n_, -1);
    encl_.assign(n_, -1);
    arg_of_.assign(n_, -1);
    guarded_.assign(n_, false);
    if_of_.assign(n_, -1);
    std::vector<int> stack;     // open loop ids / -2 for If
    std::vector<int> if_stack;  // instr index of open Ifs
    size_t n_globals = 0;
    for (int i = 0; i < n_; ++i) {
      const ughip_instr& in = I_[i];
      int cur = -1;
      for (int k = (int)stack.size() - 1; k >= 0; --k)
        if (stack[k] >= 0) {
          cur = stack[k];
          break;
        }
      encl_[i] = cur;
      guarded_[i] = !if_stack.empty();
      if_of_[i] = if_stack.empty() ? -1 : if_stack.back();
      if (in.dtype < 0 || in.dtype > UGHIP_I64) fail("bad dtype at " + std::to_string(i));
      switch (in.op) {
        case UGHIP_I_DEFINE_ACC:
        case UGHIP_I_CONST:
          if (!in.a.is_const) fail("DefineAcc/Const without a constant at " + std::to_string(i));
          check_a(in.a, i);
          vt_[i] = {true, false, false, in.a.dtype};
          break;
        case UGHIP_I_DEFINE_GLOBAL: {
          if (in.n >= s_.n_args) fail("DefineGlobal index out of range");
          if (s_.args[in.n].var != (uint32_t)i) fail("kernel args do not match DefineGlobal lines");
          if (!s_.args[in.n].is_ptr) fail("non-pointer arguments are not supported yet");
          arg_of_[i] = (int)in.n;
          vt_[i] = {true, true, false, in.dtype};
          ++n_globals;
          break;
        }
        case UGHIP_I_DEFINE_LOCAL:
          if (in.n == 0 || in.n * dtype_size(in.dtype) > 160 * 1024) fail("DefineLocal size out of range");
          vt_[i] = {true, true, true, in.dtype};
          break;
        case UGHIP_I_SPECIAL:
          if (in.sub != UGHIP_SPECIAL_THREAD_IDX && in.sub != UGHIP_SPECIAL_BLOCK_IDX) fail("bad Special");
          vt_[i] = {true, false, false, UGHIP_I32};
          break;
        case UGHIP_I_UNARY:
          if (in.sub < UGHIP_U_ID || in.sub > UGHIP_U_CAST) fail("bad unary op");
          check_a(in.a, i);
          vt_[i] = {true, false, false, in.dtype};
          break;
        case UGHIP_I_BINARY:
          if (in.sub < UGHIP_B_ADD || in.sub > UGHIP_B_MAX) fail("bad binary op");
          check_a(in.a, i);
          check_a(in.b, i);
          vt_[i] = {true, false, false, in.dtype};
          break;
        case UGHIP_I_RANGE: {
          check_a(in.a, i);
          check_a(in.b, i);
          if (in.n == 0) fail("Range with step 0");
          if ((int)in.v >= n_ || (int)in.v <= i || I_[in.v].op != UGHIP_I_END_RANGE || (int)I_[in.v].v != i)
            fail("Range/EndRange mismatch at " + std::to_string(i));
          LoopInfo li;
          li.begin = i;
          li.end = (int)in.v;
          li.parent = cur;
          li.depth = cur < 0 ? 0 : loops_[cur].depth + 1;
          li.step = (i64)in.n;
          i64 lo, up;
          if (const_int(in.a, &lo) && const_int(in.b, &up)) {
            li.cb = true;
            li.lo = lo;
            li.up = up;
            li.trip = up > lo ? (up - lo + li.step - 1) / li.step : 0;
          }
          loop_id_[i] = (int)loops_.size();
          loops_.push_back(li);
          stack.push_back(loop_id_[i]);
          vt_[i] = {true, false, false, UGHIP_I32};
          break;
        }
        case UGHIP_I_END_RANGE:
          if (stack.empty() || stack.back() < 0 || loops_[stack.back()].end != i || (int)in.v != loops_[stack.back()].begin)
            fail("unmatched EndRange");
          stack.pop_back();
          encl_[i] = loops_[loop_id_[in.v]].parent;
          break;
        case UGHIP_I_LOAD:
          check_a(in.a, i);
          if ((int)in.v >= i || !vt_[in.v].ptr) fail("Load from a non-pointer at " + std::to_string(i));
          vt_[i] = {true, false, false, in.dtype};
          break;
        case UGHIP_I_STORE:
          check_a(in.a, i);
          check_a(in.b, i);
          if ((int)in.v >= i || !vt_[in.v].ptr) fail("Store to a non-pointer at " + std::to_string(i));
          break;
        case UGHIP_I_ASSIGN:
          check_a(in.a, i);
          if ((int)in.v >= i || !vt_[in.v].valid || vt_[in.v].ptr) fail("Assign to a non-value at " + std::to_string(i));
          break;
        case UGHIP_I_IF:
          check_a(in.a, i);
          if ((int)in.v >= n_ || (int)in.v <= i || I_[in.v].op != UGHIP_I_END_IF) fail("If/EndIf mismatch");
          stack.push_back(-2);
          if_stack.push_back(i);
          break;
        case UGHIP_I_END_IF:
          if (stack.empty() || stack.back() != -2 || (int)I_[if_stack.back()].v != i) fail("unmatched EndIf");
          stack.pop_back();
          if_stack.pop_back();
          break;
        case UGHIP_I_BARRIER: break;
        case UGHIP_I_REDUCE_LOCAL:
          if (in.sub < UGHIP_R_SUM || in.sub > UGHIP_R_MIN) fail("bad reduce op");
          check_a(in.a, i);
          vt_[i] = {true, false, false, in.dtype};
          break;
        default: fail("unknown instruction kind " + std::to_string(in.op));
      }
    }
    if (!stack.empty()) fail("unmatched Range");
    if (n_globals != s_.n_args) fail("args/DefineGlobal count mismatch");
    if (loops_.size() > 60) fail("too many loops");
  }

  uint64_t open_mask(int i) const {
    uint64_t m = 0;
    for (int l = encl_[i]; l >= 0; l = loops_[l].parent) m |= 1ull << l;
    return m;
  }

  uint64_t use_dep(const ughip_a& a, uint64_t open) const { return a.is_const ? 0 : (dep_[a.var] & open); }

  void compute_deps() {
    dep_.assign(n_, 0);
    for (int pass = 0; pass < 8; ++pass) {
      bool changed = false;
      for (int i = 0; i < n_; ++i) {
        const ughip_instr& in = I_[i];
        uint64_t open = open_mask(i);
        uint64_t d = 0;
        switch (in.op) {
          case UGHIP_I_UNARY:
          case UGHIP_I_LOAD:
          case UGHIP_I_REDUCE_LOCAL: d = use_dep(in.a, open); break;
          case UGHIP_I_BINARY: d = use_dep(in.a, open) | use_dep(in.b, open); break;
          case UGHIP_I_RANGE: d = use_dep(in.a, open) | use_dep(in.b, open) | (1ull << loop_id_[i]); break;
          case UGHIP_I_STORE: d = use_dep(in.a, open) | use_dep(in.b, open); break;
          case UGHIP_I_ASSIGN: {
            uint64_t add = use_dep(in.a, open) | (open & ~open_mask((int)in.v));
            if ((dep_[in.v] | add) != dep_[in.v]) {
              dep_[in.v] |= add;
              changed = true;
            }
            d = dep_[in.v];
            break;
          }
          default: break;
        }
        // A Range variable is visible (and varies) inside its own loop.
        if ((dep_[i] | d) != dep_[i]) {
          dep_[i] |= d;
          changed = true;
        }
      }
      if (!changed) break;
    }
  }

  // ---- integer intervals and per-argument extent ----------------------------------------
  static Itv itv_binop(int op, const Itv& a, const Itv& b) {
    Itv r;
    if (!a.known || !b.known) return r;
    auto mul = [](i64 x, i64 y) { return x * y; };
    switch (op) {
      case UGHIP_B_ADD: r = {true, a.lo + b.lo, a.hi + b.hi}; break;
      case UGHIP_B_SUB: r = {true, a.lo - b.hi, a.hi - b.lo}; break;
      case UGHIP_B_MUL: {
        i64 c[4] = {mul(a.lo, b.lo), mul(a.lo, b.hi), mul(a.hi, b.lo), mul(a.hi, b.hi)};
        r = {true, *std::min_element(c, c + 4), *std::max_element(c, c + 4)};
        break;
      }
      case UGHIP_B_DIV:
        if (b.lo > 0 && a.lo >= 0) r = {true, a.lo / b.hi, a.hi / b.lo};
        break;
      case UGHIP_B_MOD:
        if (b.lo > 0 && a.lo >= 0) r = {true, 0, std::min(a.hi, b.hi - 1)};
        break;
      case UGHIP_B_MIN: r = {true, std::min(a.lo, b.lo), std::min(a.hi, b.hi)}; break;
      case UGHIP_B_MAX: r = {true, std::max(a.lo, b.lo), std::max(a.hi, b.hi)}; break;
    }
    if (r.known && (std::llabs(r.lo) > (1ll << 40) || std::llabs(r.hi) > (1ll << 40))) r.known = false;
    return r;
  }

  Itv itv_of(const ughip_a& a) const {
    if (a.is_const) {
      if (a.dtype == UGHIP_I32 || a.dtype == UGHIP_I64) return {true, a.i, a.i};
      return {};
    }
    return itv_[a.var];
  }

  void compute_intervals(bool gpu_style) {
    itv_.assign(n_, Itv());
    for (int i = 0; i < n_; ++i) {
      const ughip_instr& in = I_[i];
      bool int_result = vt_[i].valid && !vt_[i].ptr && (vt_[i].dtype == UGHIP_I32 || vt_[i].dtype == UGHIP_I64);
      switch (in.op) {
        case UGHIP_I_CONST:
          if (int_result) itv_[i] = {true, in.a.i, in.a.i};
          break;
        case UGHIP_I_SPECIAL:
          if (gpu_style) {
            i64 hi = in.sub == UGHIP_SPECIAL_THREAD_IDX ? (i64)std::max(1u, s_.block_dim) - 1 : (i64)std::max(1u, s_.grid_dim) - 1;
            itv_[i] = {true, 0, hi};
          }
          break;
        case UGHIP_I_RANGE: {
          Itv lo = itv_of(in.a), up = itv_of(in.b);
          if (lo.known && up.known) itv_[i] = {true, lo.lo, std::max(lo.lo, up.hi - 1)};
          break;
        }
        case UGHIP_I_BINARY:
          if (int_result) itv_[i] = itv_binop(in.sub, itv_of(in.a), itv_of(in.b));
          break;
        case UGHIP_I_UNARY:
          if (int_result) {
            Itv a = itv_of(in.a);
            if (a.known && in.sub == UGHIP_U_ID) itv_[i] = a;
            if (a.known && in.sub == UGHIP_U_NEG) itv_[i] = {true, -a.hi, -a.lo};
          }
          break;
        default: break;
      }
    }
    // Accumulators that are reassigned have no static interval.
    for (int i = 0; i < n_; ++i)
      if (I_[i].op == UGHIP_I_ASSIGN) itv_[I_[i].v].known = false;
  }


  // ---- what an enclosing If says about the integers of the kernel ------------------------------
  // The SSA has no comparison: a guard is an integer that is non-zero when the body runs, built from Sub / Max / Min / Mul
  // (`max(n - i, 0)`, `min(a, b)` or `a * b` of two such).  constrain(v, want) records that value v lies in `want`
  // inside the body and pushes that through the defining instruction to its operands; every step is a necessary
  // condition of the guard being taken, never a guess, so intervals only shrink.
  static constexpr i64 kInf = 1ll << 41;
  static Itv meet(const Itv& a, const Itv& b) {
    if (!a.known) return b;
    if (!b.known) return a;
    return {true, std::max(a.lo, b.lo), std::min(a.hi, b.hi)};
  }
  void constrain(std::map<int, Itv>& over, const ughip_a& a, Itv want, int depth) const {
    if (a.is_const || depth > 16) return;
    const int v = (int)a.var;
    if (!itv_[v].known) return;  // reassigned accumulators, floats: nothing static to narrow
    Itv cur = over.count(v) ? over[v] : itv_[v];
    Itv now = meet(cur, want);
    if (now.lo == cur.lo && now.hi == cur.hi && over.count(v)) return;
    over[v] = now;
    const ughip_instr& d = I_[v];
    auto of = [&](const ughip_a& x) { return x.is_const || !over.count((int)x.var) ? itv_of(x) : over.at((int)x.var); };
    if (d.op == UGHIP_I_UNARY && d.sub == UGHIP_U_ID) constrain(over, d.a, now, depth + 1);
    if (d.op == UGHIP_I_UNARY && d.sub == UGHIP_U_NEG) constrain(over, d.a, {true, -now.hi, -now.lo}, depth + 1);
    if (d.op != UGHIP_I_BINARY) return;
    const Itv x = of(d.a), y = of(d.b);
    if (!x.known || !y.known) return;
    switch (d.sub) {
      case UGHIP_B_ADD:
        constrain(over, d.a, {true, now.lo - y.hi, now.hi - y.lo}, depth + 1);
        constrain(over, d.b, {true, now.lo - x.hi, now.hi - x.lo}, depth + 1);
        break;
      case UGHIP_B_SUB:  // v = a - b
        constrain(over, d.a, {true, now.lo + y.lo, now.hi + y.hi}, depth + 1);
        constrain(over, d.b, {true, x.lo - now.hi, x.hi - now.lo}, depth + 1);
        break;
      case UGHIP_B_MAX:  // v >= lo with one side below lo: the other side is at least lo; v <= hi holds for both
        constrain(over, d.a, {true, y.hi < now.lo ? now.lo : -kInf, now.hi}, depth + 1);
        constrain(over, d.b, {true, x.hi < now.lo ? now.lo : -kInf, now.hi}, depth + 1);
        break;
      case UGHIP_B_MIN:
        constrain(over, d.a, {true, now.lo, y.lo > now.hi ? now.hi : kInf}, depth + 1);
        constrain(over, d.b, {true, now.lo, x.lo > now.hi ? now.hi : kInf}, depth + 1);
        break;
      case UGHIP_B_MUL:  // a product of two non-negative integers is non-zero only if both are
        if (x.lo >= 0 && y.lo >= 0 && now.lo >= 1) {
          constrain(over, d.a, {true, 1, kInf}, depth + 1);
          constrain(over, d.b, {true, 1, kInf}, depth + 1);
        }
        break;
      default: break;
    }
  }

  // Interval of the offset `off` of the access at instruction `at`, given that every If around it was taken.
  Itv offset_under_guards(int at, const ughip_a& off) const {
    if (off.is_const) return itv_of(off);
    std::map<int, Itv> over;
    for (int f = if_of_[at]; f >= 0; f = if_of_[f]) {
      const Itv c = itv_of(I_[f].a);
      if (!c.known) continue;
      if (c.lo >= 0) constrain(over, I_[f].a, {true, 1, kInf}, 0);
      else if (c.hi <= 0) constrain(over, I_[f].a, {true, -kInf, -1}, 0);
    }
    if (over.empty()) return itv_of(off);
    // forward again from the first narrowed value: integers computed from narrowed ones narrow with them
    std::vector<Itv> t(itv_.begin(), itv_.begin() + at);
    for (auto& kv : over)
      if (kv.first < at) t[kv.first] = kv.second;
    auto of = [&](const ughip_a& x) -> Itv { return x.is_const ? itv_of(x) : ((int)x.var < at ? t[x.var] : Itv()); };
    for (int i = over.begin()->first + 1; i < at; ++i) {
      if (!itv_[i].known) continue;
      const ughip_instr& in = I_[i];
      Itv r;
      if (in.op == UGHIP_I_BINARY) r = itv_binop(in.sub, of(in.a), of(in.b));
      else if (in.op == UGHIP_I_UNARY && in.sub == UGHIP_U_ID) r = of(in.a);
      else if (in.op == UGHIP_I_UNARY && in.sub == UGHIP_U_NEG) {
        const Itv a = of(in.a);
        if (a.known) r = {true, -a.hi, -a.lo};
      } else continue;
      if (r.known) t[i] = meet(t[i], r);
    }
    const Itv o = t[off.var];
    if (o.known && o.lo > o.hi) return {true, 0, -1};  // the guard can never be taken: the access touches nothing
    return o;
  }

  // Is instruction i inside a loop that provably never runs?
  bool dead(int i) const {
    for (int l = encl_[i]; l >= 0; l = loops_[l].parent)
      if (loops_[l].cb && loops_[l].trip == 0) return true;
    return false;
  }

  void compute_bounds() {
    bool live_store = false, any_store = false;
    for (int i = 0; i < n_; ++i) {
      const ughip_instr& in = I_[i];
      if (in.op != UGHIP_I_LOAD && in.op != UGHIP_I_STORE) continue;
      int a = arg_of_[in.v];
      if (a < 0) continue;  // LDS
      if (in.op == UGHIP_I_STORE) {
        out_.arg_written[a] = 1;
        any_store = true;
      }
      if (dead(i)) continue;
      if (in.op == UGHIP_I_STORE) live_store = true;
      // An access under an If may be exactly what the guard keeps in range (a grid rounded up to the block size with
      // `if (max(n - i, 0))` around the store).  Where the guard's value pins integers of the kernel (see narrow_by_guards)
      // the offset is re-evaluated under those narrower intervals; any other condition leaves the full requirement.
      Itv o = guarded_[i] ? offset_under_guards(i, in.a) : itv_of(in.a);
      if (!o.known || o.lo < 0)
        out_.min_len[a] = -1;
      else if (out_.min_len[a] >= 0)
        out_.min_len[a] = std::max(out_.min_len[a], o.hi + 1);
    }
    // Every store sits in a zero-trip loop: the launch is a no-op (zero-sized tensors,
    // ug-cuda/src/runtime.rs:269-277).
    if (any_store && !live_store) out_.empty_launch = true;
  }

  // ---- affine forms over loop variables ----------------------------------------------------
  Aff aff_of(const ughip_a& a) const {
    if (a.is_const) {
      Aff r;
      if (a.dtype == UGHIP_I32 || a.dtype == UGHIP_I64) {
        r.ok = true;
        r.c = a.i;
      }
      return r;
    }
    return aff_[a.var];
  }

  void compute_affine() {
    aff_.assign(n_, Aff());
    for (int i = 0; i < n_; ++i) {
      const ughip_instr& in = I_[i];
      bool int_result = vt_[i].valid && !vt_[i].ptr && (vt_[i].dtype == UGHIP_I32 || vt_[i].dtype == UGHIP_I64);
      if (!int_result) continue;
      Aff r;
      switch (in.op) {
        case UGHIP_I_CONST:
          r.ok = true;
          r.c = in.a.i;
          break;
        case UGHIP_I_RANGE:
          r.ok = true;
          r.t[loop_id_[i]] = 1;
          break;
        case UGHIP_I_UNARY:
          if (in.sub == UGHIP_U_ID) r = aff_of(in.a);
          break;
        case UGHIP_I_BINARY: {
          Aff a = aff_of(in.a), b = aff_of(in.b);
          if (!a.ok || !b.ok) break;
          if (in.sub == UGHIP_B_ADD || in.sub == UGHIP_B_SUB) {
            i64 sg = in.sub == UGHIP_B_ADD ? 1 : -1;
            r = a;
            r.c += sg * b.c;
            for (auto& kv : b.t) r.t[kv.first] += sg * kv.second;
          } else if (in.sub == UGHIP_B_MUL) {
            const Aff* k = a.t.empty() ? &a : (b.t.empty() ? &b : nullptr);
            const Aff* o = k == &a ? &b : &a;
            if (!k) break;
            r = *o;
            r.c *= k->c;
            for (auto& kv : r.t) kv.second *= k->c;
          } else if (a.t.empty() && b.t.empty() && b.c != 0 && (in.sub == UGHIP_B_DIV || in.sub == UGHIP_B_MOD)) {
            r.ok = true;
            r.c = in.sub == UGHIP_B_DIV ? a.c / b.c : a.c % b.c;
          }
          break;
        }
        default: break;
      }
      for (auto it = r.t.begin(); it != r.t.end();) it = it->second == 0 ? r.t.erase(it) : std::next(it);
      aff_[i] = r;
    }
    for (int i = 0; i < n_; ++i)
      if (I_[i].op == UGHIP_I_ASSIGN) aff_[I_[i].v].ok = false;
  }

  // ---- text emission -----------------------------------------------------------------------
  static std::string var(int i) { return "v" + std::to_string(i); }

  static std::string f32_lit(float f) {
    if (std::isinf(f)) return f > 0 ? "__builtin_inff()" : "(-__builtin_inff())";
    if (std::isnan(f)) fail("cannot use nan in const");
    char buf[64];
    snprintf(buf, sizeof buf, "%.9g", (double)f);
    std::string s(buf);
    if (s.find('.') == std::string::npos && s.find('e') == std::string::npos && s.find("inf") == std::string::npos) s += ".0";
    return s + "f";
  }

  static std::string const_lit(const ughip_a& a) {
    switch (a.dtype) {
      case UGHIP_I32: return a.i < 0 ? "(" + std::to_string(a.i) + ")" : std::to_string(a.i);
      case UGHIP_I64: return "(" + std::to_string(a.i) + "LL)";
      case UGHIP_F32: return f32_lit(a.f);
      case UGHIP_F16: return "((_Float16)" + f32_lit(a.f) + ")";
      case UGHIP_BF16: return "((__bf16)" + f32_lit(a.f) + ")";
    }
    fail("bad const dtype");
  }

  // Parametric mode: 32-bit integer constants are not printed but read from a by-value kernel
  // argument (`ug_k.v[i]`).  Two kernels that differ only in such constants -- the same op on
  // another shape, e.g. the KV length growing by one per decode step -- then share their source
  // text and therefore the compiled code object.
  bool parametric_ = false;
  mutable std::vector<int> kparams_;
  std::string kparam(i64 v) const {
    kparams_.push_back((int)v);
    return "ug_k.v[" + std::to_string(kparams_.size() - 1) + "]";
  }
  std::string lit(const ughip_a& a) const {
    if (parametric_ && a.dtype == UGHIP_I32) return kparam(a.i);
    return const_lit(a);
  }

  std::string opnd(const ughip_a& a) const { return a.is_const ? lit(a) : var((int)a.var); }

  static const char* reduce_functor(int op) { return op == UGHIP_R_SUM ? "ug_sum" : (op == UGHIP_R_MAX ? "ug_max" : "ug_min"); }

  static std::string identity_lit(int op, int dt) {
    ughip_a a{};
    a.is_const = 1;
    a.dtype = (uint8_t)dt;
    if (op == UGHIP_R_SUM) {
      a.i = 0;
      a.f = 0.f;
    } else if (is_float(dt)) {
      a.f = op == UGHIP_R_MAX ? -INFINITY : INFINITY;
    } else if (dt == UGHIP_I32) {
      a.i = op == UGHIP_R_MAX ? INT32_MIN : INT32_MAX;
    } else {
      return op == UGHIP_R_MAX ? "(-9223372036854775807LL - 1)" : "9223372036854775807LL";
    }
    return const_lit(a);
  }

  // One statement for instruction i (loops open/close a brace).
  std::string stmt(int i) const {
    const ughip_instr& in = I_[i];
    std::string ty = vt_[i].valid && !vt_[i].ptr ? dtype_c_name(vt_[i].dtype) : "";
    std::ostringstream o;
    switch (in.op) {
      case UGHIP_I_DEFINE_GLOBAL: return "";
      case UGHIP_I_DEFINE_LOCAL: o << "__shared__ " << dtype_c_name(in.dtype) << " " << var(i) << "[" << in.n << "];"; break;
      case UGHIP_I_DEFINE_ACC:
      case UGHIP_I_CONST: o << ty << " " << var(i) << " = " << lit(in.a) << ";"; break;
      case UGHIP_I_SPECIAL:
        o << "const int " << var(i) << " = " << (in.sub == UGHIP_SPECIAL_THREAD_IDX ? "(int)threadIdx.x" : "(int)blockIdx.x") << ";";
        break;
      case UGHIP_I_UNARY: {
        std::string a = opnd(in.a);
        bool f32 = in.dtype == UGHIP_F32;
        auto fn = [&](const char* name) {
          // 16-bit floats go through f32 math; ints are converted like the C backend does.
          if (f32) return std::string(name) + "f(" + a + ")";
          return "(" + ty + ")" + name + "f((float)(" + a + "))";
        };
        std::string e;
        switch (in.sub) {
          case UGHIP_U_ID: e = a; break;
          case UGHIP_U_EXP: e = fn("exp"); break;
          case UGHIP_U_SIN: e = fn("sin"); break;
          case UGHIP_U_COS: e = fn("cos"); break;
          case UGHIP_U_SQRT: e = fn("sqrt"); break;
          case UGHIP_U_NEG: e = "-(" + a + ")"; break;
          case UGHIP_U_CAST: e = "(" + ty + ")(" + a + ")"; break;
        }
        o << ty << " " << var(i) << " = " << e << ";";
        break;
      }
      case UGHIP_I_BINARY: {
        std::string a = opnd(in.a), b = opnd(in.b), e;
        bool fl = is_float(in.dtype);
        switch (in.sub) {
          case UGHIP_B_ADD: e = a + " + " + b; break;
          case UGHIP_B_SUB: e = a + " - " + b; break;
          case UGHIP_B_MUL: e = a + " * " + b; break;
          case UGHIP_B_DIV: e = a + " / " + b; break;
          case UGHIP_B_MOD: e = fl ? "fmodf((float)(" + a + "), (float)(" + b + "))" : a + " % " + b; break;
          case UGHIP_B_MIN:
            e = fl ? "fminf((float)(" + a + "), (float)(" + b + "))" : "((" + a + ") < (" + b + ") ? (" + a + ") : (" + b + "))";
            break;
          case UGHIP_B_MAX:
            e = fl ? "fmaxf((float)(" + a + "), (float)(" + b + "))" : "((" + a + ") > (" + b + ") ? (" + a + ") : (" + b + "))";
            break;
        }
        o << ty << " " << var(i) << " = " << e << ";";
        break;
      }
      case UGHIP_I_RANGE:
        o << "for (int " << var(i) << " = " << opnd(in.a) << "; " << var(i) << " < " << opnd(in.b) << "; " << var(i)
          << " += " << in.n << ") {";
        break;
      case UGHIP_I_END_RANGE:
      case UGHIP_I_END_IF: o << "}"; break;
      case UGHIP_I_IF: o << "if (" << opnd(in.a) << ") {"; break;
      case UGHIP_I_LOAD:
        if (nt_loads_) o << ty << " " << var(i) << " = __builtin_nontemporal_load(&" << var((int)in.v) << "[" << opnd(in.a) << "]);";
        else o << ty << " " << var(i) << " = " << var((int)in.v) << "[" << opnd(in.a) << "];";
        break;
      case UGHIP_I_ASSIGN: o << var((int)in.v) << " = " << opnd(in.a) << ";"; break;
      case UGHIP_I_STORE:
        if (nt_stores_ && arg_of_[in.v] >= 0 && (in.dtype == UGHIP_F32 || in.dtype == UGHIP_I32 || in.dtype == UGHIP_I64))
          o << "__builtin_nontemporal_store((" << dtype_c_name(in.dtype) << ")(" << opnd(in.b) << "), &" << var((int)in.v) << "[" << opnd(in.a) << "]);";
        else
          o << var((int)in.v) << "[" << opnd(in.a) << "] = " << opnd(in.b) << ";";
        break;
      case UGHIP_I_BARRIER: o << "__syncthreads();"; break;
      case UGHIP_I_REDUCE_LOCAL: {
        int dt = in.dtype;
        if (dt == UGHIP_F32 || dt == UGHIP_I32 || dt == UGHIP_I64)
          o << ty << " " << var(i) << " = ug_block_reduce_dyn<" << reduce_functor(in.sub) << ", " << ty << ">(" << opnd(in.a) << ");";
        else
          o << ty << " " << var(i) << " = (" << ty << ")ug_block_reduce_dyn<" << reduce_functor(in.sub) << ", float>((float)(" << opnd(in.a)
            << "));";
        break;
      }
    }
    return o.str();
  }

  std::string signature(bool scratch) const {
    std::ostringstream o;
    for (size_t a = 0; a < s_.n_args; ++a) {
      if (a) o << ", ";
      o << (out_.arg_written[a] ? "" : "const ") << dtype_c_name(s_.args[a].dtype) << "* __restrict__ " << var((int)s_.args[a].var);
    }
    if (scratch) {
      if (s_.n_args) o << ", ";
      o << "void* __restrict__ ug_part_raw";
    }
    return o.str();
  }

  void emit_range(std::ostringstream& o, int from, int to, int indent) const {
    int depth = indent;
    for (int i = from; i <= to; ++i) {
      int op = I_[i].op;
      if (op == UGHIP_I_END_RANGE || op == UGHIP_I_END_IF) --depth;
      std::string s = stmt(i);
      if (!s.empty()) o << std::string(2 * depth, ' ') << s << "\n";
      if (op == UGHIP_I_RANGE || op == UGHIP_I_IF) ++depth;
    }
  }

  void emit_literal(unsigned grid, unsigned block) {
    if (block > 1024) fail("block_dim > 1024");
    std::ostringstream o;
    o << kPrelude << "\nextern \"C\" __global__ void __launch_bounds__(" << block << ") " << entry_ << "(" << signature(false) << ") {\n";
    emit_range(o, 0, n_ - 1, 1);
    o << "}\n";
    out_.source = o.str();
    out_.strategy = UGHIP_STRAT_LITERAL;
    out_.grid = grid;
    out_.block = block;
    out_.lds_bytes = s_.shared_mem;
  }

  // ---- re-parallelisation --------------------------------------------------------------------
  std::vector<int> chain_;       // loop ids, outermost first
  std::vector<Region> regions_;
  std::vector<Item> items_;

  bool loop_has(int l, int op) const {
    for (int i = loops_[l].begin; i <= loops_[l].end; ++i)
      if (I_[i].op == op) return true;
    return false;
  }

  bool loop_assigns_outer(int l) const {
    for (int i = loops_[l].begin; i <= loops_[l].end; ++i)
      if (I_[i].op == UGHIP_I_ASSIGN && (int)I_[i].v < loops_[l].begin) return true;
    return false;
  }

  bool references(const ughip_a& a, int v) const { return !a.is_const && (int)a.var == v; }

  // `DefineAcc; Range; ...; t = fold(acc, x); Assign acc = t; EndRange` with the accumulator
  // touched nowhere else inside the loop.
  bool match_region(int l, Region* r) const {
    const LoopInfo& L = loops_[l];
    if (!L.cb || L.step < 1) return false;
    int assign = -1;
    for (int i = L.begin + 1; i < L.end; ++i) {
      if (I_[i].op != UGHIP_I_ASSIGN) continue;
      if ((int)I_[i].v > L.begin) continue;  // local to the loop body
      if (assign >= 0 || encl_[i] != l) return false;
      assign = i;
    }
    if (assign < 0) return false;
    int acc = (int)I_[assign].v;
    if (I_[acc].op != UGHIP_I_DEFINE_ACC) return false;
    if (I_[assign].a.is_const) return false;
    int fold = (int)I_[assign].a.var;
    if (fold <= L.begin || I_[fold].op != UGHIP_I_BINARY || encl_[fold] != l) return false;
    const ughip_instr& f = I_[fold];
    int rop;
    if (f.sub == UGHIP_B_ADD) rop = UGHIP_R_SUM;
    else if (f.sub == UGHIP_B_MAX) rop = UGHIP_R_MAX;
    else if (f.sub == UGHIP_B_MIN) rop = UGHIP_R_MIN;
    else return false;
    bool lhs = references(f.a, acc), rhs = references(f.b, acc);
    if (lhs == rhs) return false;
    int dt = vt_[acc].dtype;
    if (f.dtype != dt || !(dt == UGHIP_F32 || dt == UGHIP_I32 || dt == UGHIP_I64)) return false;
    // The fold result must feed only the Assign; the accumulator only the fold.
    for (int i = L.begin; i <= L.end; ++i) {
      if (i == fold || i == assign) continue;
      const ughip_instr& in = I_[i];
      if (references(in.a, acc) || references(in.b, acc) || references(in.a, fold) || references(in.b, fold)) return false;
      if ((in.op == UGHIP_I_LOAD || in.op == UGHIP_I_STORE) && ((int)in.v == acc)) return false;
    }
    r->range = L.begin;
    r->end = L.end;
    r->acc = acc;
    r->fold = fold;
    r->assign = assign;
    r->op = rop;
    r->acc_is_lhs = lhs;
    r->trip = L.trip;
    r->loop = l;
    return true;
  }

  uint64_t span_deps(int from, int to, uint64_t mask) const {
    uint64_t d = 0;
    for (int i = from; i <= to; ++i) d |= dep_[i];
    return d & mask;
  }

  bool plan_auto() {
    // 1. the chain of parallel loops that encloses every Store.
    std::vector<int> stores;
    for (int i = 0; i < n_; ++i)
      if (I_[i].op == UGHIP_I_STORE) stores.push_back(i);
    if (stores.empty()) return false;
    int level = -1;
    for (;;) {
      int cand = -1, count = 0;
      bool store_here = false;
      for (int i = 0; i < n_; ++i) {
        if (encl_[i] != level) continue;
        if (I_[i].op == UGHIP_I_STORE) store_here = true;
        if (I_[i].op == UGHIP_I_RANGE && loop_has(loop_id_[i], UGHIP_I_STORE)) {
          cand = loop_id_[i];
          ++count;
        }
      }
      if (store_here || count != 1) break;
      const LoopInfo& L = loops_[cand];
      if (!L.cb || loop_assigns_outer(cand)) break;
      // Nothing may follow the loop at its own level (values defined inside would be out of scope).
      bool tail = false;
      int level_end = level < 0 ? n_ - 1 : loops_[level].end - 1;
      for (int i = L.end + 1; i <= level_end; ++i)
        if (I_[i].op != UGHIP_I_END_RANGE) tail = true;
      if (tail) break;
      chain_.push_back(cand);
      level = cand;
    }
    for (int st : stores)
      if (encl_[st] != level) return false;
    uint64_t chain_mask = 0;
    for (int l : chain_) chain_mask |= 1ull << l;
    for (int l : chain_)
      if (loops_[l].trip == 0) {
        out_.empty_launch = true;
      }
    // 2. stored buffers are never read, stores hit distinct addresses across the chain.
    for (int i = 0; i < n_; ++i)
      if (I_[i].op == UGHIP_I_LOAD && arg_of_[I_[i].v] >= 0 && out_.arg_written[arg_of_[I_[i].v]]) return false;
    for (int st : stores) {
      Aff a = aff_of(I_[st].a);
      if (!a.ok) return false;
      std::vector<std::pair<i64, i64>> ce;  // |coef|, extent
      for (int l : chain_) {
        if (loops_[l].trip <= 1) continue;
        auto it = a.t.find(l);
        if (it == a.t.end()) return false;
        ce.push_back({std::llabs(it->second) * loops_[l].step, loops_[l].trip});
      }
      for (auto& kv : a.t)
        if (!(chain_mask >> kv.first & 1)) return false;
      std::sort(ce.begin(), ce.end());
      for (size_t k = 0; k + 1 < ce.size(); ++k)
        if (ce[k + 1].first < ce[k].first * ce[k].second) return false;
    }
    // 3. items in program order.
    for (int i = 0; i < n_;) {
      const ughip_instr& in = I_[i];
      if (in.op == UGHIP_I_RANGE) {
        int l = loop_id_[i];
        if (chain_mask >> l & 1) {
          ++i;
          continue;
        }
        Item it;
        it.idx = i;
        it.end = loops_[l].end;
        Region r;
        if (match_region(l, &r)) {
          it.kind = 1;
          it.region = (int)regions_.size();
          regions_.push_back(r);
        } else {
          it.kind = 2;
        }
        it.deps = span_deps(i, it.end, chain_mask);
        items_.push_back(it);
        i = it.end + 1;
        continue;
      }
      if (in.op == UGHIP_I_END_RANGE) {
        ++i;
        continue;
      }  // closes a chain loop
      if (in.op != UGHIP_I_DEFINE_GLOBAL) {
        Item it;
        it.idx = it.end = i;
        it.deps = dep_[i] & chain_mask;
        items_.push_back(it);
      }
      ++i;
    }
    // 4. rows and columns.
    uint64_t row_mask = 0;
    for (const Item& it : items_)
      if (it.kind == 1) row_mask |= it.deps;
    i64 total = 1;
    for (int l : chain_) total *= std::max<i64>(loops_[l].trip, 0);
    if (total >= (1ll << 31)) return false;
    if (out_.empty_launch) {
      emit_literal(1, 1);  // valid source, never launched
      return true;
    }
    if (regions_.empty()) {
      emit_elementwise(total);
      return true;
    }
    std::vector<int> rows, cols;
    i64 nr = 1, nc = 1;
    for (int l : chain_) {
      if (row_mask >> l & 1) {
        rows.push_back(l);
        nr *= loops_[l].trip;
      } else {
        cols.push_back(l);
        nc *= loops_[l].trip;
      }
    }
    // Which variable walks memory with stride 1 inside the reductions?
    bool red_unit = false, row_unit = false, any_dep = false;
    for (const Region& r : regions_)
      for (int i = r.range; i <= r.end; ++i) {
        if (I_[i].op != UGHIP_I_LOAD) continue;
        Aff a = aff_of(I_[i].a);
        if (!a.ok) continue;
        auto it = a.t.find(r.loop);
        if (it != a.t.end()) {
          any_dep = true;
          if (std::llabs(it->second) * loops_[r.loop].step == 1) red_unit = true;
        }
        for (int l : rows) {
          auto jt = a.t.find(l);
          if (jt != a.t.end() && std::llabs(jt->second) * loops_[l].step == 1 && loops_[l].trip > 1) row_unit = true;
        }
      }
    i64 max_trip = 0;
    for (const Region& r : regions_) max_trip = std::max(max_trip, r.trip);
    if (any_dep && !red_unit && row_unit && nr >= 64) {
      emit_row_thread(rows, cols, nr, nc);
      return true;
    }
    if (regions_.size() == 1 && nr <= 64 && max_trip >= (1 << 16)) {
      emit_row_block(rows, cols, nr, nc, /*grid_reduce=*/true);
      return true;
    }
    emit_row_block(rows, cols, nr, nc, false);
    return true;
  }

  // `const int v<loop> = lo + digit * step;` for each loop of `ls`.  `group` counts groups of
  // `vec` consecutive iterations of the innermost (fastest) loop; `ug_u` selects inside the group,
  // which keeps the addresses of the unrolled copies visibly consecutive for the compiler.
  void emit_decode(std::ostringstream& o, const std::vector<int>& ls, const std::string& group, int vec, int indent) const {
    std::string pad(2 * indent, ' ');
    if (ls.empty()) return;
    o << pad << "int ug_r = " << group << ";\n";
    for (int k = (int)ls.size() - 1; k >= 0; --k) {
      const LoopInfo& L = loops_[ls[k]];
      bool inner = k == (int)ls.size() - 1;
      i64 radix = inner ? L.trip / vec : L.trip;
      // one spelling of the radix per loop, so the % and / below share it (one parameter slot)
      std::string rs = !k ? "" : (parametric_ ? kparam(radix) : std::to_string(radix));
      std::string digit = k == 0 ? "ug_r" : "(ug_r % " + rs + ")";
      if (inner && vec > 1) digit = "(" + digit + " * " + std::to_string(vec) + " + ug_u)";
      o << pad << "const int " << var(L.begin) << " = ";
      if (parametric_) {
        o << kparam(L.lo) << " + " << digit << " * " << kparam(L.step);
      } else {
        if (L.lo) o << L.lo << " + ";
        o << digit;
        if (L.step != 1) o << " * " << L.step;
      }
      o << ";\n";
      if (k) o << pad << "ug_r /= " << rs << ";\n";
    }
  }

  static int pick_vec(i64 extent, i64 threads) {
    // the last wave of several may be partly idle: full-width loads still win over keeping it busy
    if (extent % 4 == 0 && (extent >= threads * 4 || (threads > 64 && extent > (threads - 64) * 4))) return 4;
    if (extent % 2 == 0 && extent >= threads * 2) return 2;
    return 1;
  }

  void emit_items(std::ostringstream& o, bool want_cols, uint64_t col_mask, int indent, bool guard_row_stores, int tpr, bool one_thread) const {
    for (const Item& it : items_) {
      bool is_col = (it.deps & col_mask) != 0;
      if (is_col != want_cols) continue;
      if (it.kind == 1 && !one_thread) {
        if (is_col) fail("internal: reduction depends on a column loop");
        emit_region(o, regions_[it.region], indent, tpr);
      } else if (it.kind == 0 && I_[it.idx].op == UGHIP_I_STORE && guard_row_stores && !is_col) {
        o << std::string(2 * indent, ' ') << "if (ug_t == 0) { " << stmt(it.idx) << " }\n";
      } else {
        emit_range(o, it.idx, it.end, indent);
      }
    }
  }

  // Statements of a reduction loop body with the fold redirected to the thread-local partial.
  void emit_reduce_body(std::ostringstream& o, const Region& r, int indent) const {
    std::string ty = dtype_c_name(vt_[r.acc].dtype);
    std::string fn = reduce_functor(r.op);
    std::string part = "ug_p" + std::to_string(r.acc);
    int depth = indent;
    for (int i = r.range + 1; i < r.end; ++i) {
      if (i == r.assign) continue;
      int op = I_[i].op;
      if (op == UGHIP_I_END_RANGE) --depth;
      std::string pad(2 * depth, ' ');
      if (i == r.fold) {
        const ughip_instr& f = I_[i];
        std::string x = opnd(r.acc_is_lhs ? f.b : f.a);
        o << pad << part << " = " << fn << "::f(" << part << ", (" << ty << ")(" << x << "));\n";
        continue;
      }
      std::string s = stmt(i);
      if (!s.empty()) o << pad << s << "\n";
      if (op == UGHIP_I_RANGE) ++depth;
    }
  }

  // Cooperative reduction by the `tpr` threads that share a row; afterwards every one of them
  // holds the folded accumulator in v<acc>.
  void emit_region(std::ostringstream& o, const Region& r, int indent, int tpr) const {
    std::string pad(2 * indent, ' ');
    const LoopInfo& L = loops_[r.loop];
    std::string ty = dtype_c_name(vt_[r.acc].dtype);
    int vec = pick_vec(L.trip, tpr);
    std::string part = "ug_p" + std::to_string(r.acc);
    o << pad << ty << " " << part << " = " << identity_lit(r.op, vt_[r.acc].dtype) << ";\n";
    o << pad << "for (int ug_i = ug_t * " << vec << "; ug_i < " << L.trip << "; ug_i += " << tpr * vec << ") {\n";
    o << pad << "#pragma unroll\n";
    o << pad << "  for (int ug_u = 0; ug_u < " << vec << "; ++ug_u) {\n";
    o << pad << "    const int " << var(L.begin) << " = ";
    if (L.lo) o << L.lo << " + ";
    o << "(ug_i + ug_u)";
    if (L.step != 1) o << " * " << L.step;
    o << ";\n";
    emit_reduce_body(o, r, indent + 2);
    o << pad << "  }\n" << pad << "}\n";
    emit_region_finish(o, r, indent, tpr);
  }

  void emit_region_finish(std::ostringstream& o, const Region& r, int indent, int tpr) const {
    std::string pad(2 * indent, ' ');
    std::string ty = dtype_c_name(vt_[r.acc].dtype);
    std::string fn = reduce_functor(r.op);
    std::string part = "ug_p" + std::to_string(r.acc);
    int nw = (tpr + 63) / 64;
    o << pad << part << " = ug_block_reduce<" << fn << ", " << ty << ", " << nw << ">(" << part << ");\n";
    o << pad << var(r.acc) << " = " << fn << "::f(" << var(r.acc) << ", " << part << ");\n";
  }

  void emit_elementwise(i64 total) {
    const int block = 256;
    i64 inner = chain_.empty() ? 1 : loops_[chain_.back()].trip;
    int vec = inner % 4 == 0 ? 4 : (inner % 2 == 0 ? 2 : 1);
    if (total < (i64)block * vec * 64) vec = 1;  // small problem: favour more threads
    i64 groups = total / vec;
    // Small kernels (the per-token elementwise work of a decode step, whose shapes follow the KV
    // length) are emitted parametric so that a new shape does not mean a new hiprtc compile; large
    // ones keep their constants, which lets the compiler strength-reduce the index arithmetic.
    parametric_ = total <= (1 << 20) && !ughip::tune_on(ughip::TUNE_NO_PARAMETRIC);
    kparams_.clear();
    // Whole 128-bit groups are stored past the cache: nothing in the launch reads them back (stored buffers are never loaded
    // here), and the next kernel would find them in another XCD's L2 at best.  SwiGLU [512, 5632]: 4.6 -> 3.6 us, [16384, 5632]
    // 184 -> 179 us.  Not for the row kernels: their stores do not merge under the hint (RMSNorm [8192, 2048]: 20.8 -> 31.6 us).
    nt_stores_ = vec == 4 && !ughip::tune_on(ughip::TUNE_NO_NT_STORES);
    std::ostringstream b;
    b << "  const int ug_g = (int)blockIdx.x * " << block << " + (int)threadIdx.x;\n";
    b << "  if (ug_g >= " << (parametric_ ? kparam(groups) : std::to_string(groups)) << ") return;\n";
    // Items that depend on no loop are computed once per thread, ahead of the unrolled part.
    uint64_t all = 0;
    for (int l : chain_) all |= 1ull << l;
    emit_items(b, false, all, 1, false, 1, true);
    b << "#pragma unroll\n  for (int ug_u = 0; ug_u < " << vec << "; ++ug_u) {\n";
    emit_decode(b, chain_, "ug_g", vec, 2);
    emit_items(b, true, all, 2, false, 1, true);
    b << "  }\n}\n";
    std::ostringstream o;
    o << kPrelude << "\n";
    std::string sig = signature(false);
    if (parametric_) {
      o << "struct ug_params { int v[" << kparams_.size() << "]; };\n";
      sig += std::string(sig.empty() ? "" : ", ") + "const ug_params ug_k";
      out_.kparams = kparams_;
    }
    o << "extern \"C\" __global__ void __launch_bounds__(" << block << ") " << entry_ << "(" << sig << ") {\n" << b.str();
    parametric_ = false;
    nt_stores_ = false;
    out_.source = o.str();
    out_.strategy = UGHIP_STRAT_ELEMENTWISE;
    out_.block = block;
    out_.grid = (unsigned)((groups + block - 1) / block);
  }

  void emit_row_thread(const std::vector<int>& rows, const std::vector<int>& cols, i64 nr, i64 nc) {
    const int block = 256;
    uint64_t col_mask = 0;
    for (int l : cols) col_mask |= 1ull << l;
    std::ostringstream o;
    o << kPrelude << "\nextern \"C\" __global__ void __launch_bounds__(" << block << ") " << entry_ << "(" << signature(false) << ") {\n";
    o << "  const int ug_row = (int)blockIdx.x * " << block << " + (int)threadIdx.x;\n";
    o << "  if (ug_row >= " << nr << ") return;\n";
    o << "  {\n";
    emit_decode(o, rows, "ug_row", 1, 2);
    emit_items(o, false, col_mask, 2, false, 1, true);
    o << "    for (int ug_c = 0; ug_c < " << nc << "; ++ug_c) {\n";
    emit_decode(o, cols, "ug_c", 1, 3);
    emit_items(o, true, col_mask, 3, false, 1, true);
    o << "    }\n  }\n}\n";
    out_.source = o.str();
    out_.strategy = UGHIP_STRAT_ROW_THREAD;
    out_.block = block;
    out_.grid = (unsigned)((nr + block - 1) / block);
  }

  static unsigned tune_u(ughip::TuneKey k, unsigned dflt) {
    long long v;
    return ughip::tune_get(k, &v) && v > 0 ? (unsigned)v : dflt;
  }

  void emit_row_block(const std::vector<int>& rows, const std::vector<int>& cols, i64 nr, i64 nc, bool grid_reduce) {
    uint64_t col_mask = 0;
    for (int l : cols) col_mask |= 1ull << l;
    i64 width = nc;
    for (const Region& r : regions_) width = std::max(width, r.trip);
    int tpr;  // threads that share a row
    if (grid_reduce) {
      tpr = (int)tune_u(ughip::TUNE_GRID_REDUCE_THREADS, 256);
    } else if (width <= 256) {
      tpr = 64;
    } else {
      // one 128-bit slab per thread where the row allows it: whole waves, not a power of two of them (768 columns
      // take 3 waves; rounding up to 4 left a quarter of the threads idle and halved the width of every load)
      tpr = (int)std::min<i64>(1024, ((width + 3) / 4 + 63) / 64 * 64);
    }
    int rows_per_block = tpr == 64 ? 4 : 1;
    if (nr < rows_per_block) rows_per_block = 1;
    int block = tpr * rows_per_block;
    std::ostringstream o;
    o << kPrelude << "\nextern \"C\" __global__ void __launch_bounds__(" << block << ") " << entry_ << "(" << signature(grid_reduce) << ") {\n";
    o << "  const int ug_t = (int)threadIdx.x % " << tpr << ";\n";
    unsigned nb = 1;
    if (grid_reduce) {
      const Region& r = regions_[0];
      int vec = pick_vec(r.trip, tpr);
      i64 per_block_iter = (i64)tpr * vec;
      // Measured on MI355X: one workgroup of 256 threads per CU (256 of them), each thread walking >= 4 slabs with
      // four 128-bit loads per operand in flight.  Two per CU (512) is as fast on some boxes and 6-9 % slower on
      // others, in bursts and behind seconds of the same launches alike (2 x 64 MiB: 21.4 against 23.4 us per step
      // sustained; 2 x 512 MiB: 152 against 162 us); 128 or 384 leave CUs idle for half a round.
      i64 want = (r.trip + per_block_iter * 4 - 1) / (per_block_iter * 4);
      unsigned cap = std::max<i64>(1, 256 / nr);
      nb = (unsigned)std::max<i64>(1, std::min<i64>(want, cap));
      nb = tune_u(ughip::TUNE_GRID_REDUCE_BLOCKS, nb);
      o << "  const int ug_row = (int)blockIdx.x / " << nb << ";\n";
      o << "  const int ug_blk = (int)blockIdx.x % " << nb << ";\n";
    } else {
      o << "  const int ug_row = (int)blockIdx.x * " << rows_per_block << " + (int)threadIdx.x / " << tpr << ";\n";
      if (rows_per_block > 1) o << "  if (ug_row >= " << nr << ") return;\n";
    }
    o << "  {\n";
    emit_decode(o, rows, "ug_row", 1, 2);
    if (!grid_reduce) {
      emit_items(o, false, col_mask, 2, true, tpr, false);
    } else {
      // Stage 1 (this kernel): every workgroup folds its slabs of the reduction and stores one
      // partial.  Stage 2 (`<entry>_fin`, one workgroup per row, launched right behind on the same
      // stream) folds the partials in index order and carries on with the rest of the row.  The
      // kernel boundary is the only synchronisation: no fences, no atomics, same bits every run.
      const Region& r = regions_[0];
      std::string ty = dtype_c_name(vt_[r.acc].dtype);
      std::string fn = reduce_functor(r.op);
      std::string part = "ug_p" + std::to_string(r.acc);
      std::vector<const Item*> before, after;
      bool seen = false;
      for (const Item& it : items_) {
        if ((it.deps & col_mask) != 0) continue;
        if (it.kind == 1) {
          seen = true;
          continue;
        }
        (seen ? after : before).push_back(&it);
      }
      // Only what the reduction body needs has to run in stage 1, but the row-invariant prefix is
      // a handful of scalar instructions: emit it in both stages.
      for (const Item* it : before) emit_range(o, it->idx, it->end, 2);
      o << "    " << ty << "* __restrict__ ug_part = (" << ty << "*)ug_part_raw;\n";
      // The first stage streams its operands once: loads that do not claim cache lines (measured on
      // 2 x 64 MiB: 22.0 -> 20.6 us).  Kernels that come back to a row (softmax, norms) and plain
      // copies lose with them (6.8 -> 5.9 TB/s for a 64 MiB copy), so nothing else uses them.
      nt_loads_ = !ughip::tune_on(ughip::TUNE_NO_NT_LOADS);
      emit_region_partial(o, r, 2, tpr, nb);
      nt_loads_ = false;
      o << "    if (ug_t == 0) ug_part[ug_row * " << nb << " + ug_blk] = " << part << ";\n";
      o << "  }\n}\n";
      // ---- stage 2
      o << "\nextern \"C\" __global__ void __launch_bounds__(" << tpr << ") " << entry_ << "_fin(" << signature(true) << ") {\n";
      o << "  const int ug_t = (int)threadIdx.x;\n";
      o << "  const int ug_row = (int)blockIdx.x;\n";
      o << "  {\n";
      emit_decode(o, rows, "ug_row", 1, 2);
      for (const Item* it : before) emit_range(o, it->idx, it->end, 2);
      o << "    const " << ty << "* __restrict__ ug_part = (const " << ty << "*)ug_part_raw;\n";
      o << "    " << ty << " " << part << " = " << identity_lit(r.op, vt_[r.acc].dtype) << ";\n";
      o << "    for (int ug_i = ug_t; ug_i < " << nb << "; ug_i += " << tpr << ")\n";
      o << "      " << part << " = " << fn << "::f(" << part << ", ug_part[ug_row * " << nb << " + ug_i]);\n";
      emit_region_finish(o, r, 2, tpr);
      for (const Item* it : after) {
        if (it->kind == 0 && I_[it->idx].op == UGHIP_I_STORE)
          o << "    if (ug_t == 0) { " << stmt(it->idx) << " }\n";
        else
          emit_range(o, it->idx, it->end, 2);
      }
      out_.scratch_part_bytes = (size_t)nr * nb * dtype_size(vt_[r.acc].dtype);
      out_.entry2 = entry_ + "_fin";
      out_.grid2 = (unsigned)nr;
      out_.block2 = (unsigned)tpr;
    }
    bool any_col = false;
    for (const Item& it : items_) any_col |= (it.deps & col_mask) != 0;
    if (any_col) {
      i64 inner = cols.empty() ? 1 : loops_[cols.back()].trip;
      int vec = (inner % 4 == 0 && pick_vec(nc, tpr) == 4) ? 4 : 1;
      o << "    for (int ug_c = ug_t; ug_c < " << nc / vec << "; ug_c += " << tpr << ") {\n";
      o << "#pragma unroll\n";
      o << "      for (int ug_u = 0; ug_u < " << vec << "; ++ug_u) {\n";
      emit_decode(o, cols, "ug_c", vec, 4);
      emit_items(o, true, col_mask, 4, false, tpr, false);
      o << "      }\n    }\n";
    }
    o << "  }\n}\n";
    out_.source = o.str();
    out_.strategy = grid_reduce ? UGHIP_STRAT_GRID_REDUCE : UGHIP_STRAT_ROW_BLOCK;
    out_.block = (unsigned)block;
    out_.grid = grid_reduce ? (unsigned)(nr * nb) : (unsigned)((nr + rows_per_block - 1) / rows_per_block);
  }

  // First stage of a grid-wide reduction: workgroup `ug_blk` of `nb` takes every nb-th slab.
  void emit_region_partial(std::ostringstream& o, const Region& r, int indent, int tpr, unsigned nb) const {
    std::string pad(2 * indent, ' ');
    const LoopInfo& L = loops_[r.loop];
    std::string ty = dtype_c_name(vt_[r.acc].dtype);
    std::string fn = reduce_functor(r.op);
    int vec = pick_vec(L.trip, tpr);
    std::string part = "ug_p" + std::to_string(r.acc);
    o << pad << ty << " " << part << " = " << identity_lit(r.op, vt_[r.acc].dtype) << ";\n";
    // 32-bit indices (ssa offsets are i32 anyway) keep the `vec` unrolled accesses visibly
    // consecutive, so they merge into one 128-bit load; a constant trip count lets the compiler
    // batch the loads of several slabs before the first use.
    const i64 stride = (i64)nb * tpr * vec;
    const i64 iters = (L.trip + stride - 1) / stride;
    const bool tail = L.trip % stride != 0;
    const bool wide = L.trip + stride >= (1ll << 31);
    const char* it_ty = wide ? "long long" : "int";
    o << pad << "const " << it_ty << " ug_base = ((" << it_ty << ")ug_blk * " << tpr << " + ug_t) * " << vec << ";\n";
    o << pad << "#pragma unroll " << (iters >= 4 ? 4 : (int)iters) << "\n";
    o << pad << "for (int ug_it = 0; ug_it < " << iters << "; ++ug_it) {\n";
    o << pad << "  const " << it_ty << " ug_i = ug_base + (" << it_ty << ")ug_it * " << stride << (wide ? "LL" : "") << ";\n";
    if (tail) o << pad << "  if (ug_i >= " << L.trip << ") break;\n";
    o << pad << "#pragma unroll\n";
    o << pad << "  for (int ug_u = 0; ug_u < " << vec << "; ++ug_u) {\n";
    o << pad << "    const int " << var(L.begin) << " = ";
    if (L.lo) o << L.lo << " + ";
    o << "(int)(ug_i + ug_u)";
    if (L.step != 1) o << " * " << L.step;
    o << ";\n";
    emit_reduce_body(o, r, indent + 2);
    o << pad << "  }\n" << pad << "}\n";
    o << pad << part << " = ug_block_reduce<" << fn << ", " << ty << ", " << (tpr + 63) / 64 << ">(" << part << ");\n";
  }
};

}  // namespace

Lowered lower_ssa(const ughip_ssa& ssa, const std::string& entry, bool as_written) {
  if (!ssa.instrs || (!ssa.args && ssa.n_args)) throw std::runtime_error("ssa lowering: null instrs/args");
  Lowering l(ssa, entry, as_written);
  return l.run();
}

}  // namespace ughip
