// ORACLE -- TEST INFRASTRUCTURE ONLY.  Nothing under ug_amd/ may include, link or call this.
//
// CPU restatement of ug's CPU backend, the reference every HIP result is compared with:
//   * gen_c():      ssa::Kernel -> C text, rule for rule after ug-core/src/cpu_code_gen.rs:68-186
//                   (one statement per instruction, `int` indices, fmin/fmax for every dtype,
//                   expf/sqrtf/sinf/cosf, `%` for Mod, +-inf spelled `1. / 0.`);
//   * CpuDevice:    ug-core/src/cpu_runtime.rs:251-359 -- zero-filled allocation (:255-264),
//                   compile = gcc -shared -lm -O3 -march=native -ffast-math -fomit-frame-pointer
//                   (:476-488) + dlopen, run with at most 5 pointer arguments (:288-334),
//                   exact-copy slices with dtype/len checks (:376-412);
//   * matmul:       stride rules of cpu_runtime.rs:527-619.  The arithmetic of the reference
//                   lives in the un-vendored `gemm` 0.18.0 crate; here it is a plain f32
//                   multiply-accumulate in k order per output element (F32, and F16 widened to
//                   f32 with one final rounding).  PARITY UNPINNED beyond
//                   the reference's own `mm` test (common_tests.rs:15-22): the tests therefore
//                   also compare against an f64 product with a k*eps bound.
// Pinned by: the golden vectors of ug-core/tests/{basic_tests,lb_tests,cpu_tests}.rs and
// ug-core/src/common_tests.rs (tests/golden/), closed forms (tests/test_oracle_*.py).
#include <dlfcn.h>
#include <sys/wait.h>
#include <unistd.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <thread>

#include "oracle.h"

namespace ug_oracle {

using namespace ug;

namespace {

const char* c_type(int dt) {
  switch (dt) {
    case UGHIP_BF16: return "__bf16";
    case UGHIP_F16: return "_Float16";  // __fp16 on arm, _Float16 on x86
    case UGHIP_F32: return "float";
    case UGHIP_I32: return "int";
    case UGHIP_I64: return "long long";
  }
  bail("unknown dtype");
}

std::string v(uint32_t id) { return "__var" + std::to_string(id); }

// cpu_code_gen.rs:14-28: shortest decimal that round-trips, always with a '.', an exponent or inf.
std::string fmt_f32(float x) {
  if (std::isnan(x)) return "0. / 0.";
  if (std::isinf(x)) return x > 0 ? "1. / 0." : "-1. / 0.";
  char buf[64];
  for (int prec = 1; prec <= 9; ++prec) {
    snprintf(buf, sizeof buf, "%.*g", prec, (double)x);
    if (strtof(buf, nullptr) == x) break;
  }
  std::string s(buf);
  if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
  return s;
}

std::string c_const(const ughip_a& a) {
  switch (a.dtype) {
    case UGHIP_I32:
    case UGHIP_I64: return std::to_string(a.i);
    default: return fmt_f32(a.f);
  }
}

std::string c_a(const ughip_a& a) { return a.is_const ? c_const(a) : v(a.var); }

}  // namespace

// cpu_code_gen.rs:68-186
std::string gen_c(const std::string& func_name, const ssa::Kernel& kernel) {
  for (const auto& in : kernel.instrs)
    if (in.op == UGHIP_I_REDUCE_LOCAL) bail("TODO: add the reduce code if needed");
  std::ostringstream w;
  w << "#include<math.h>\n";
  w << "void " << func_name << "(\n";
  for (size_t i = 0; i < kernel.args.size(); ++i) {
    const auto& a = kernel.args[i];
    std::string ty = a.is_ptr ? std::string(c_type(a.dtype)) + "*" : std::string(c_type(a.dtype));
    w << "  " << ty << " " << v(a.var) << (i + 1 == kernel.args.size() ? "" : ",") << "\n";
  }
  w << ") {\n";
  size_t depth = 0;
  for (size_t id = 0; id < kernel.instrs.size(); ++id) {
    const ssa::Instr& in = kernel.instrs[id];
    std::string var_id = v((uint32_t)id);
    std::string indent(2 * depth + 2, ' ');
    switch (in.op) {
      case UGHIP_I_DEFINE_GLOBAL: break;
      case UGHIP_I_DEFINE_LOCAL: w << indent << "__shared__ " << c_type(in.dtype) << " " << var_id << "[" << in.n << "];\n"; break;
      case UGHIP_I_DEFINE_ACC:
      case UGHIP_I_CONST: w << indent << c_type(in.a.dtype) << " " << var_id << " = " << c_const(in.a) << ";\n"; break;
      case UGHIP_I_IF:
        w << indent << "if (" << c_a(in.a) << ") {\n";
        ++depth;
        break;
      case UGHIP_I_RANGE:
        w << indent << "for (int " << var_id << " = " << c_a(in.a) << "; " << var_id << " < " << c_a(in.b) << "; " << var_id << "+=" << in.n
          << ") {\n";
        ++depth;
        break;
      case UGHIP_I_END_IF:
      case UGHIP_I_END_RANGE:
        if (depth == 0) bail("unmatched EndRange");
        --depth;
        w << std::string(2 * depth + 2, ' ') << "}\n";
        break;
      case UGHIP_I_LOAD: w << indent << c_type(in.dtype) << " " << var_id << " = " << v(in.v) << "[" << c_a(in.a) << "];\n"; break;
      case UGHIP_I_ASSIGN: w << indent << v(in.v) << " = " << c_a(in.a) << ";\n"; break;
      case UGHIP_I_STORE: w << indent << v(in.v) << "[" << c_a(in.a) << "] = " << c_a(in.b) << ";\n"; break;
      case UGHIP_I_BINARY: {
        std::string l = c_a(in.a), r = c_a(in.b), e;
        switch (in.sub) {
          case UGHIP_B_ADD: e = l + " + " + r; break;
          case UGHIP_B_MUL: e = l + " * " + r; break;
          case UGHIP_B_SUB: e = l + " - " + r; break;
          case UGHIP_B_DIV: e = l + " / " + r; break;
          case UGHIP_B_MIN: e = "fmin(" + l + ", " + r + ")"; break;
          case UGHIP_B_MAX: e = "fmax(" + l + ", " + r + ")"; break;
          case UGHIP_B_MOD: e = l + " % " + r; break;
        }
        w << indent << c_type(in.dtype) << " " << var_id << " = " << e << ";\n";
        break;
      }
      case UGHIP_I_UNARY: {
        std::string op;
        switch (in.sub) {
          case UGHIP_U_SQRT: op = "sqrtf"; break;
          case UGHIP_U_EXP: op = "expf"; break;
          case UGHIP_U_SIN: op = "sinf"; break;
          case UGHIP_U_COS: op = "cosf"; break;
          case UGHIP_U_NEG: op = "-"; break;
          case UGHIP_U_ID: op = ""; break;
          case UGHIP_U_CAST: op = std::string("(") + c_type(in.dtype) + ")"; break;
        }
        w << indent << c_type(in.dtype) << " " << var_id << " = " << op << "(" << c_a(in.a) << ");\n";
        break;
      }
      case UGHIP_I_SPECIAL:
        if (in.sub == UGHIP_SPECIAL_THREAD_IDX) bail("thread-id is currently not supported in the cpu backend");
        bail("block-id is currently not supported in the cpu backend");
      case UGHIP_I_BARRIER: break;  // single thread: nothing to do
      case UGHIP_I_REDUCE_LOCAL: bail("unreachable");
      default: bail("unknown instruction");
    }
  }
  w << "}\n";
  if (depth > 0) bail("unmatched Range");
  return w.str();
}

// ---- storage ------------------------------------------------------------------------------------
CpuSlice::CpuSlice(DType dt, size_t len) : dtype_(dt), len_(len), bytes_(len * size_in_bytes(dt), 0) {}

void CpuSlice::copy_host_to_device(const void* src, DType dtype, size_t len) {
  if (len != len_) bail("dtoh len mismatch, dst " + std::to_string(len_) + ", len " + std::to_string(len));
  if (dtype != dtype_) bail(std::string("htod dtype mismatch, dst ") + dtype_str(dtype_) + ", src " + dtype_str(dtype));
  if (len) std::memcpy(bytes_.data(), src, bytes_.size());
}

void CpuSlice::copy_device_to_host(void* dst, DType dtype, size_t len) const {
  if (len != len_) bail("dtoh len mismatch, dst " + std::to_string(len) + ", len " + std::to_string(len_));
  if (dtype != dtype_) bail(std::string("dtoh dtype mismatch, dst ") + dtype_str(dtype) + ", src " + dtype_str(dtype_));
  if (len) std::memcpy(dst, bytes_.data(), bytes_.size());
}

CpuSlice& cpu_slice(Slice& s) {
  CpuSlice* c = dynamic_cast<CpuSlice*>(&s);
  if (!c) bail("slice does not belong to the cpu device");
  return *c;
}
const CpuSlice& cpu_slice(const Slice& s) {
  const CpuSlice* c = dynamic_cast<const CpuSlice*>(&s);
  if (!c) bail("slice does not belong to the cpu device");
  return *c;
}

// ---- compile / run --------------------------------------------------------------------------------
struct CpuFunc : Func {
  std::string func_name, c_code;
  void* lib = nullptr;
  void* sym = nullptr;
  ~CpuFunc() override {
    if (lib) dlclose(lib);
  }
};

static int run_gcc(const std::string& c_path, const std::string& so_path, std::string* output) {
  // cpu_runtime.rs:476-488
  std::string cmd = "gcc '" + c_path + "' -shared -lm -O3 -march=native -ffast-math -fomit-frame-pointer -o '" + so_path + "' 2>&1";
  FILE* p = popen(cmd.c_str(), "r");
  if (!p) bail("cannot start gcc");
  char buf[512];
  while (fgets(buf, sizeof buf, p)) *output += buf;
  int status = pclose(p);
  return WIFEXITED(status) ? WEXITSTATUS(status) : 1;
}

std::shared_ptr<Func> CpuDevice::compile_c(const std::string& c_code, const std::string& func_name) {
  const char* tmp = getenv("TMPDIR");
  std::string dir = tmp && *tmp ? tmp : "/tmp";
  std::string c_path = dir + "/" + func_name + ".c", so_path = dir + "/" + func_name + ".so";
  {
    std::ofstream f(c_path);
    f << c_code;
  }
  std::string output;
  int rc = run_gcc(c_path, so_path, &output);
  auto func = std::make_shared<CpuFunc>();
  func->func_name = func_name;
  func->c_code = c_code;
  std::string err;
  if (rc != 0) {
    err = "compilation failed\nstdout:\n" + output;
  } else {
    func->lib = dlopen(so_path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!func->lib) err = std::string("dlopen: ") + dlerror();
    else if (!(func->sym = dlsym(func->lib, func_name.c_str()))) err = "symbol not found: " + func_name;
  }
  if (!getenv("UG_KEEP_TMP")) {
    unlink(c_path.c_str());
    unlink(so_path.c_str());
  }
  if (!err.empty()) bail(err);
  return func;
}

// cpu_runtime.rs:274-286
std::shared_ptr<Func> CpuDevice::compile(const ssa::Kernel& kernel, const std::string* name) {
  static std::atomic<size_t> kernel_id{1};
  size_t kid = kernel_id.fetch_add(1);
  std::string func_name = name ? "ugc_" + *name + "_" + std::to_string(getpid()) + "_" + std::to_string(kid)
                               : "ugc_" + std::to_string(getpid()) + "_" + std::to_string(kid);
  return compile_c(gen_c(func_name, kernel), func_name);
}

// cpu_runtime.rs:288-334
void CpuDevice::run(Func& f, const std::vector<Slice*>& args) {
  CpuFunc* cf = dynamic_cast<CpuFunc*>(&f);
  if (!cf) bail("func does not belong to the cpu device");
  void* p[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
  if (args.size() > 5) bail("unsupported number of args for kernel " + std::to_string(args.size()));
  for (size_t i = 0; i < args.size(); ++i) p[i] = cpu_slice(*args[i]).data();
  switch (args.size()) {
    case 0: reinterpret_cast<void (*)()>(cf->sym)(); break;
    case 1: reinterpret_cast<void (*)(void*)>(cf->sym)(p[0]); break;
    case 2: reinterpret_cast<void (*)(void*, void*)>(cf->sym)(p[0], p[1]); break;
    case 3: reinterpret_cast<void (*)(void*, void*, void*)>(cf->sym)(p[0], p[1], p[2]); break;
    case 4: reinterpret_cast<void (*)(void*, void*, void*, void*)>(cf->sym)(p[0], p[1], p[2], p[3]); break;
    case 5: reinterpret_cast<void (*)(void*, void*, void*, void*, void*)>(cf->sym)(p[0], p[1], p[2], p[3], p[4]); break;
  }
}

std::string func_c_code(const Func& f) {
  const CpuFunc* cf = dynamic_cast<const CpuFunc*>(&f);
  return cf ? cf->c_code : std::string();
}

std::unique_ptr<Slice> CpuDevice::allocate_uninit(DType dtype, size_t len) { return std::unique_ptr<Slice>(new CpuSlice(dtype, len)); }

// ---- matmul (cpu_runtime.rs:514-619) -----------------------------------------------------------------
namespace {
size_t skip(const Layout& l, size_t dflt, const char* which) {
  const auto& st = l.strides();
  size_t rank = st.size();
  if (rank == 2) return dflt;
  if (rank == 3) return st[0];
  if (rank == 4) {
    if (st[0] == st[1] * l.dims()[1]) return st[1];
    if (l.dims()[0] == 1) return st[1];
    if (l.dims()[1] == 1) return st[0];
  }
  bail(std::string("MatMulUnexpectedStriding: non-contiguous ") + which);
}

unsigned num_threads() {
  // utils.rs:3-20: RAYON_NUM_THREADS, else all cores.
  const char* e = getenv("RAYON_NUM_THREADS");
  if (e && *e) {
    long n = strtol(e, nullptr, 10);
    if (n > 0) return (unsigned)n;
  }
  unsigned hc = std::thread::hardware_concurrency();
  return hc ? std::min(hc, 64u) : 1;
}
}  // namespace

void CpuDevice::matmul(Slice& dst_s, const Slice& lhs_s, const Slice& rhs_s, size_t b, size_t m, size_t n, size_t k, const Layout& lhs_l,
                       const Layout& rhs_l) {
  CpuSlice& dst = cpu_slice(dst_s);
  const CpuSlice& lhs = cpu_slice(lhs_s);
  const CpuSlice& rhs = cpu_slice(rhs_s);
  // cpu_runtime.rs:345-356: F16 and F32 only.
  const bool all_f32 = dst.dtype() == DType::F32 && lhs.dtype() == DType::F32 && rhs.dtype() == DType::F32;
  const bool all_f16 = dst.dtype() == DType::F16 && lhs.dtype() == DType::F16 && rhs.dtype() == DType::F16;
  if (!all_f32 && !all_f16)
    bail(std::string("incorrect dtypes for matmul, dst: ") + dtype_str(dst.dtype()) + ", lhs: " + dtype_str(lhs.dtype()) + ", rhs: " +
         dtype_str(rhs.dtype()));
  size_t rank = lhs_l.rank();
  if (rank < 2 || rhs_l.rank() != rank) bail("matmul: unexpected layout ranks");
  // F16: operands widened to f32, f32 accumulation in k order, one rounding to f16 at the end
  // (the arithmetic of the gemm crate's f16 path is unpinned here, like its f32 path).
  std::vector<float> a32, b32, c32;
  if (all_f16) {
    const uint16_t* ha = reinterpret_cast<const uint16_t*>(lhs.data());
    const uint16_t* hb = reinterpret_cast<const uint16_t*>(rhs.data());
    a32.resize(lhs.len());
    b32.resize(rhs.len());
    for (size_t i = 0; i < lhs.len(); ++i) a32[i] = f16_bits_to_f32(ha[i]);
    for (size_t i = 0; i < rhs.len(); ++i) b32[i] = f16_bits_to_f32(hb[i]);
    c32.resize(b * m * n);
  }
  const float* A = (all_f16 ? a32.data() : reinterpret_cast<const float*>(lhs.data())) + lhs_l.offset();
  const float* B = (all_f16 ? b32.data() : reinterpret_cast<const float*>(rhs.data())) + rhs_l.offset();
  float* C = all_f16 ? c32.data() : reinterpret_cast<float*>(dst.data());
  size_t a_cs = lhs_l.strides()[rank - 1], a_rs = lhs_l.strides()[rank - 2];
  size_t b_cs = rhs_l.strides()[rank - 1], b_rs = rhs_l.strides()[rank - 2];
  size_t a_skip = skip(lhs_l, m * k, "lhs"), b_skip = skip(rhs_l, n * k, "rhs"), c_skip = m * n;
  if (dst.len() < b * m * n) bail("matmul: dst too short");
  size_t rows = b * m;
  if (rows == 0 || n == 0) return;
  unsigned nt = (unsigned)std::min<size_t>(num_threads(), std::max<size_t>(1, rows * n * k / 65536));
  // Work items are (row, column chunk) so that a single-row product (decode) still uses every core.
  size_t chunks = rows >= nt ? 1 : std::min<size_t>(n, (nt + rows - 1) / rows);
  size_t chunk = (n + chunks - 1) / chunks;
  size_t tasks = rows * chunks;
  auto work = [&](size_t t0, size_t t1) {
    std::vector<float> acc(chunk);
    for (size_t t = t0; t < t1; ++t) {
      size_t r = t / chunks, j0 = (t % chunks) * chunk, j1 = std::min(n, j0 + chunk);
      if (j0 >= j1) continue;
      size_t step = r / m, i = r % m;
      const float* a = A + step * a_skip + i * a_rs;
      const float* bb = B + step * b_skip;
      float* c = C + step * c_skip + i * n;
      if (b_cs == 1) {
        // row-major rhs: accumulate a row slice, k outermost (each c[j] still sums in k order)
        std::fill(acc.begin(), acc.end(), 0.f);
        for (size_t kk = 0; kk < k; ++kk) {
          float av = a[kk * a_cs];
          const float* brow = bb + kk * b_rs;
          for (size_t j = j0; j < j1; ++j) acc[j - j0] += av * brow[j];
        }
        std::memcpy(c + j0, acc.data(), (j1 - j0) * sizeof(float));
      } else {
        for (size_t j = j0; j < j1; ++j) {
          const float* bcol = bb + j * b_cs;
          float s = 0.f;
          for (size_t kk = 0; kk < k; ++kk) s += a[kk * a_cs] * bcol[kk * b_rs];
          c[j] = s;
        }
      }
    }
  };
  if (nt <= 1) {
    work(0, tasks);
  } else {
    std::vector<std::thread> ths;
    size_t per = (tasks + nt - 1) / nt;
    for (unsigned t = 0; t < nt; ++t) {
      size_t t0 = t * per, t1 = std::min(tasks, t0 + per);
      if (t0 < t1) ths.emplace_back(work, t0, t1);
    }
    for (auto& th : ths) th.join();
  }
  if (all_f16) {
    uint16_t* hc = reinterpret_cast<uint16_t*>(dst.data());
    for (size_t i = 0; i < c32.size(); ++i) hc[i] = f32_to_f16_bits(c32[i]);
  }
}

}  // namespace ug_oracle
