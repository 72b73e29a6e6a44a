// Flat C API over the host-side front-end, for ctypes (tests, bench) and other FFI callers.
// Every function returns 0 on success; ugh_last_error() holds the message otherwise.
#include "capi.h"

#include <cstdio>

#include "ug/safetensors.h"

#include <cstring>

#include "hip_device.h"
#include "llama.h"
#include "ug/lazy_buffer.h"
#include "ug/samples.h"

using namespace ug;

namespace {
thread_local std::string g_err;

template <typename F>
int guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_err = e.what();
    return 1;
  } catch (...) {
    g_err = "unknown error";
    return 1;
  }
}

DevicePtr& dev_of(void* d) {
  if (!d) bail("null device");
  return *static_cast<DevicePtr*>(d);
}
LazyBuffer& lb_of(void* p) {
  if (!p) bail("null lazy buffer");
  return *static_cast<LazyBuffer*>(p);
}
void* box(LazyBuffer lb) { return new LazyBuffer(std::move(lb)); }
Shape shape_of(const size_t* dims, size_t rank) { return Shape(std::vector<size_t>(dims, dims + rank)); }

Const const_of(int dtype, double v) {
  switch ((DType)dtype) {
    case DType::F32: return Const::f32((float)v);
    case DType::BF16: return Const::bf16((float)v);
    case DType::I32: return Const::i32((int32_t)v);
    case DType::I64: return Const::i64((int64_t)v);
    default: bail("unable to create const for this dtype");
  }
}

std::function<void(const std::vector<Slice*>&)> wrap_cb(ugh_custom_fn fn, void* user) {
  return [fn, user](const std::vector<Slice*>& vs) {
    std::vector<void*> raw(vs.begin(), vs.end());
    if (fn(user, raw.data(), raw.size())) bail("custom op callback failed");
  };
}

struct CompiledBox {
  CompiledSchedule cs;
};
}  // namespace

extern "C" {

const char* ugh_last_error(void) { return g_err.c_str(); }

// ---- devices -------------------------------------------------------------------------------
int ugh_hip_device_new(int ordinal, void** out) {
  return guard([&] { *out = new DevicePtr(std::make_shared<HipDevice>(ordinal)); });
}
void ugh_device_free(void* d) { delete static_cast<DevicePtr*>(d); }
int ugh_device_synchronize(void* d) {
  return guard([&] { dev_of(d)->synchronize(); });
}
const char* ugh_device_name(void* d) { return d ? (*static_cast<DevicePtr*>(d))->name() : ""; }
int ugh_device_use_grid(void* d) { return d && (*static_cast<DevicePtr*>(d))->use_grid(); }
int ugh_hip_device_set_zero_fill(void* d, int on) {
  return guard([&] {
    HipDevice* h = dynamic_cast<HipDevice*>(dev_of(d).get());
    if (!h) bail("not a hip device");
    if (ughip_device_set_zero_fill(h->raw(), on)) bail(ughip_last_error());
  });
}
void* ugh_device_raw_hip(void* d) {
  HipDevice* h = d ? dynamic_cast<HipDevice*>(static_cast<DevicePtr*>(d)->get()) : nullptr;
  return h ? h->raw() : nullptr;
}

// ---- slices / funcs at the Device boundary -----------------------------------------------------
int ugh_device_alloc(void* d, int dtype, size_t len, void** out) {
  return guard([&] { *out = dev_of(d)->allocate_uninit((DType)dtype, len).release(); });
}
// Device::convert: *done = 0 when the device does not offer it.
int ugh_device_convert(void* d, void* dst, void* src, int* done) {
  return guard([&] { *done = dev_of(d)->convert(*static_cast<Slice*>(dst), *static_cast<Slice*>(src)) ? 1 : 0; });
}
void ugh_slice_free(void* s) { delete static_cast<Slice*>(s); }
// The ughip_slice behind a slice of the HIP device (null for any other device): for callers that go to the C ABI directly.
void* ugh_slice_raw_hip(void* s) {
  HipSlice* h = s ? dynamic_cast<HipSlice*>(static_cast<Slice*>(s)) : nullptr;
  return h ? h->raw() : nullptr;
}
size_t ugh_slice_len(void* s) { return static_cast<Slice*>(s)->len(); }
int ugh_slice_dtype(void* s) { return (int)static_cast<Slice*>(s)->dtype(); }
int ugh_slice_h2d(void* s, const void* src, int dtype, size_t len) {
  return guard([&] { static_cast<Slice*>(s)->copy_host_to_device(src, (DType)dtype, len); });
}
int ugh_slice_d2h(void* s, void* dst, int dtype, size_t len) {
  return guard([&] { static_cast<Slice*>(s)->copy_device_to_host(dst, (DType)dtype, len); });
}
int ugh_device_compile(void* d, void* kernel, const char* name, void** out) {
  return guard([&] {
    std::string n = name ? name : "";
    *out = new std::shared_ptr<Func>(dev_of(d)->compile(*static_cast<ssa::Kernel*>(kernel), name ? &n : nullptr));
  });
}
void ugh_func_free(void* f) { delete static_cast<std::shared_ptr<Func>*>(f); }
int ugh_device_run(void* d, void* f, void** slices, size_t n) {
  return guard([&] {
    std::vector<Slice*> vs;
    for (size_t i = 0; i < n; ++i) vs.push_back(static_cast<Slice*>(slices[i]));
    dev_of(d)->run(**static_cast<std::shared_ptr<Func>*>(f), vs);
  });
}
void* ugh_func_raw_hip(void* f) {
  HipFunc* h = f ? dynamic_cast<HipFunc*>(static_cast<std::shared_ptr<Func>*>(f)->get()) : nullptr;
  return h ? h->raw() : nullptr;
}
int ugh_device_matmul(void* d, void* dst, void* lhs, void* rhs, size_t b, size_t m, size_t n, size_t k, size_t rank, const size_t* ldims,
                      const size_t* lstrides, size_t loff, const size_t* rdims, const size_t* rstrides, size_t roff) {
  return guard([&] {
    Layout ll, rl;
    ll.shape_ = shape_of(ldims, rank);
    ll.strides_.assign(lstrides, lstrides + rank);
    ll.offset_ = loff;
    rl.shape_ = shape_of(rdims, rank);
    rl.strides_.assign(rstrides, rstrides + rank);
    rl.offset_ = roff;
    dev_of(d)->matmul(*static_cast<Slice*>(dst), *static_cast<Slice*>(lhs), *static_cast<Slice*>(rhs), b, m, n, k, ll, rl);
  });
}

// ---- ssa kernels --------------------------------------------------------------------------------
int ugh_sample_ssa(const char* name, size_t p0, size_t p1, size_t p2, void** out) {
  return guard([&] {
    std::string n = name;
    ssa::Kernel k;
    namespace S = samples::ssa_k;
    if (n == "simple_add") k = S::simple_add(p0);
    else if (n == "simple_dotprod") k = S::simple_dotprod(p0);
    else if (n == "exp") k = S::exp(p0);
    else if (n == "exp_block") k = S::exp_block(p0, p1);
    else if (n == "softmax_barrier" || n == "softmax") k = S::softmax_barrier(p0, p1);
    else if (n == "softmax_reduce") k = S::softmax_reduce(p0, p1);
    else if (n == "softmax_block") k = S::softmax_block(p0, p1, p2);
    else bail("unknown sample kernel " + n);
    *out = new ssa::Kernel(std::move(k));
  });
}
int ugh_sample_op_ssa(const char* name, size_t p0, size_t p1, long block_axis, long thread_dim, size_t thread_block_dim, void** out) {
  return guard([&] {
    std::string n = name;
    op::Kernel k;
    if (n == "softmax") k = samples::op_softmax(p0, p1);
    else if (n == "affine") k = samples::op_affine(p0);
    else bail("unknown sample op kernel " + n);
    op::Opts opts;
    if (block_axis >= 0) opts = opts.with_block_axis((size_t)block_axis);
    if (thread_dim >= 0) opts = opts.with_thread_block((size_t)thread_dim, thread_block_dim);
    *out = new ssa::Kernel(k.lower(opts));
  });
}
int ugh_ssa_from_raw(const ughip_instr* instrs, size_t n, uint32_t grid, uint32_t block, uint32_t shared, void** out) {
  return guard([&] {
    ssa::Kernel k = ssa::Kernel::from_instrs(std::vector<ssa::Instr>(instrs, instrs + n));
    k.launch_config = LaunchConfig{grid, block, shared};
    *out = new ssa::Kernel(std::move(k));
  });
}
int ugh_ssa_wire(void* kernel, ughip_ssa* out) {
  return guard([&] { *out = static_cast<ssa::Kernel*>(kernel)->wire(); });
}
void ugh_ssa_set_launch(void* kernel, uint32_t grid, uint32_t block, uint32_t shared) {
  static_cast<ssa::Kernel*>(kernel)->launch_config = LaunchConfig{grid, block, shared};
}
void ugh_ssa_free(void* kernel) { delete static_cast<ssa::Kernel*>(kernel); }

// ---- op-level kernels and the other pieces ug-pyo3 exposes (ug-pyo3/src/lib.rs) -------------------
namespace {
size_t copy_out(const std::string& s, char* buf, size_t buf_len) {
  if (buf && buf_len) {
    size_t n = std::min(buf_len - 1, s.size());
    memcpy(buf, s.data(), n);
    buf[n] = 0;
  }
  return s.size();
}
const char* unary_name(int op) {
  static const char* n[] = {"Id", "Exp", "Sin", "Cos", "Neg", "Sqrt", "Cast"};
  return op >= 0 && op <= UGHIP_U_CAST ? n[op] : "?";
}
const char* binary_name(int op) {
  static const char* n[] = {"Add", "Sub", "Mul", "Div", "Mod", "Min", "Max"};
  return op >= 0 && op <= UGHIP_B_MAX ? n[op] : "?";
}
const char* reduce_name(int op) {
  static const char* n[] = {"Sum", "Max", "Min"};
  return op >= 0 && op <= UGHIP_R_MIN ? n[op] : "?";
}
std::string a_str(const ughip_a& a) {
  if (!a.is_const) return "Var(" + std::to_string(a.var) + ")";
  if (is_float((DType)a.dtype)) {
    char b[64];
    snprintf(b, sizeof b, "%g", (double)a.f);
    return std::string("Const(") + dtype_str((DType)a.dtype) + "(" + b + "))";
  }
  return std::string("Const(") + dtype_str((DType)a.dtype) + "(" + std::to_string((long long)a.i) + "))";
}
// One line per instruction, numbered like the reference's Debug impl (lang.rs:816-823).
std::string ssa_str(const ssa::Kernel& k) {
  std::string out;
  for (size_t i = 0; i < k.instrs.size(); ++i) {
    const ssa::Instr& in = k.instrs[i];
    char head[16];
    snprintf(head, sizeof head, "%03zu ", i);
    std::string l = head;
    const char* dt = dtype_str((DType)in.dtype);
    switch (in.op) {
      case UGHIP_I_DEFINE_ACC: l += "DefineAcc(" + a_str(in.a) + ")"; break;
      case UGHIP_I_DEFINE_GLOBAL: l += "DefineGlobal { index: " + std::to_string(in.n) + ", dtype: " + dt + " }"; break;
      case UGHIP_I_DEFINE_LOCAL: l += "DefineLocal { size: " + std::to_string(in.n) + ", dtype: " + dt + " }"; break;
      case UGHIP_I_SPECIAL: l += in.sub == UGHIP_SPECIAL_THREAD_IDX ? "Special(ThreadIdx)" : "Special(BlockIdx)"; break;
      case UGHIP_I_CONST: l += a_str(in.a); break;
      case UGHIP_I_UNARY: l += std::string("Unary { op: ") + unary_name(in.sub) + ", arg: " + a_str(in.a) + ", dtype: " + dt + " }"; break;
      case UGHIP_I_BINARY:
        l += std::string("Binary { op: ") + binary_name(in.sub) + ", lhs: " + a_str(in.a) + ", rhs: " + a_str(in.b) + ", dtype: " + dt + " }";
        break;
      case UGHIP_I_RANGE:
        l += "Range { lo: " + a_str(in.a) + ", up: " + a_str(in.b) + ", step: " + std::to_string(in.n) + ", end_idx: " + std::to_string(in.v) + " }";
        break;
      case UGHIP_I_LOAD: l += "Load { src: " + std::to_string(in.v) + ", offset: " + a_str(in.a) + ", dtype: " + dt + " }"; break;
      case UGHIP_I_ASSIGN: l += "Assign { dst: " + std::to_string(in.v) + ", src: " + a_str(in.a) + " }"; break;
      case UGHIP_I_END_RANGE: l += "EndRange { start_idx: " + std::to_string(in.v) + " }"; break;
      case UGHIP_I_IF: l += "If { cond: " + a_str(in.a) + ", end_idx: " + std::to_string(in.v) + " }"; break;
      case UGHIP_I_END_IF: l += "EndIf"; break;
      case UGHIP_I_STORE:
        l += "Store { dst: " + std::to_string(in.v) + ", offset: " + a_str(in.a) + ", value: " + a_str(in.b) + ", dtype: " + dt + " }";
        break;
      case UGHIP_I_BARRIER: l += "Barrier"; break;
      case UGHIP_I_REDUCE_LOCAL: l += std::string("ReduceLocal { op: ") + reduce_name(in.sub) + ", arg: " + a_str(in.a) + ", dtype: " + dt + " }"; break;
      default: l += "?"; break;
    }
    out += l + "\n";
  }
  return out;
}
std::string ast_str(const op::Ast& a) {
  const op::AstInner& in = *a.inner;
  switch (in.kind) {
    case op::AstInner::Load: return "Load(arg " + std::to_string(in.load_src.v) + ", " + a.shape.str() + ")";
    case op::AstInner::Const: {
      ughip_a c{};
      c.is_const = 1;
      c.dtype = (uint8_t)in.cst.dtype;
      c.i = in.cst.i;
      c.f = in.cst.f;
      return a_str(c);
    }
    case op::AstInner::Unary: return std::string(unary_name((int)in.unary_op)) + "(" + ast_str(in.arg) + ")";
    case op::AstInner::Binary: return std::string(binary_name((int)in.binary_op)) + "(" + ast_str(in.arg) + ", " + ast_str(in.rhs) + ")";
    case op::AstInner::Reduce:
      return std::string("Reduce") + reduce_name((int)in.reduce_op) + "(" + ast_str(in.arg) + ", axis " + std::to_string(in.reduce_dim) + ")";
    default: return "Layout(" + ast_str(in.arg) + " -> " + a.shape.str() + ")";
  }
}
// ssa::Kernel::flops_mem_per_thread (lang.rs:755-811)
void flops_mem(const ssa::Kernel& k, size_t* flops, size_t* mem) {
  size_t fl = 0, mm = 0, mult = 1;
  std::vector<size_t> mults;
  auto bound = [&](const ughip_a& a, const char* what) -> int64_t {
    if (a.is_const) {
      if (a.dtype != UGHIP_I32 && a.dtype != UGHIP_I64) bail(std::string("range ") + what + " is not a const i32/i64");
      return a.i;
    }
    const ssa::Instr& d = k.instrs.at(a.var);
    if (d.op != UGHIP_I_CONST || (d.a.dtype != UGHIP_I32 && d.a.dtype != UGHIP_I64)) bail(std::string("range ") + what + " is not a const");
    return d.a.i;
  };
  for (const ssa::Instr& in : k.instrs) {
    switch (in.op) {
      case UGHIP_I_LOAD:
      case UGHIP_I_STORE: mm += mult * size_in_bytes((DType)in.dtype); break;
      case UGHIP_I_RANGE: {
        mults.push_back(mult);
        int64_t lo = bound(in.a, "lo"), up = bound(in.b, "up");
        mult *= (size_t)std::max<int64_t>(up - lo, 0) / (in.n ? in.n : 1);
        break;
      }
      case UGHIP_I_END_RANGE:
        if (mults.empty()) bail("unexpected EndRange");
        mult = mults.back();
        mults.pop_back();
        break;
      case UGHIP_I_UNARY:
      case UGHIP_I_BINARY: fl += mult; break;
      default: break;
    }
  }
  *flops = fl;
  *mem = mm;
}
}  // namespace

int ugh_op_arg_new(int is_ptr, int dtype, void** out) {
  return guard([&] {
    Arg a = Arg::ptr((DType)dtype);
    a.is_ptr = is_ptr != 0;
    *out = new Arg(a);
  });
}
void ugh_op_arg_free(void* a) { delete static_cast<Arg*>(a); }
size_t ugh_op_arg_str(void* a, char* buf, size_t buf_len) {
  const Arg& x = *static_cast<Arg*>(a);
  return copy_out(std::string("Arg { id: ") + std::to_string(x.id.v) + ", type_: " + (x.is_ptr ? "Ptr(" : "Value(") + dtype_str(x.dtype) + ") }", buf, buf_len);
}
void ugh_op_ast_free(void* a) { delete static_cast<op::Ast*>(a); }
// ug-pyo3/src/lib.rs:205-214
int ugh_op_load(void* arg, const size_t* dims, size_t rank, void** out) {
  return guard([&] {
    const Arg& a = *static_cast<Arg*>(arg);
    if (!a.is_ptr) bail(std::string("unexpected dtype for load Value(") + dtype_str(a.dtype) + ")");
    *out = new op::Ast(op::load(a.id, Layout::from_shape(shape_of(dims, rank)), a.dtype));
  });
}
int ugh_op_cst_i32(int32_t v, void** out) {
  return guard([&] { *out = new op::Ast(op::cst(Const::i32(v))); });
}
int ugh_op_cst_f32(float v, void** out) {
  return guard([&] { *out = new op::Ast(op::cst(Const::f32(v))); });
}
int ugh_op_unary(void* a, int op, void** out) {
  return guard([&] { *out = new op::Ast(op::unary((UnaryOp)op, *static_cast<op::Ast*>(a))); });
}
int ugh_op_binary(int op, void* lhs, void* rhs, void** out) {
  return guard([&] { *out = new op::Ast(op::binary((BinaryOp)op, *static_cast<op::Ast*>(lhs), *static_cast<op::Ast*>(rhs))); });
}
int ugh_op_reduce(int op, void* a, size_t axis, void** out) {
  return guard([&] { *out = new op::Ast(op::reduce((ReduceOp)op, *static_cast<op::Ast*>(a), axis)); });
}
int ugh_op_broadcast(void* a, const size_t* dims, size_t rank, void** out) {
  return guard([&] { *out = new op::Ast(op::broadcast(*static_cast<op::Ast*>(a), shape_of(dims, rank))); });
}
size_t ugh_op_ast_rank(void* a) { return static_cast<op::Ast*>(a)->shape.rank(); }
void ugh_op_ast_dims(void* a, size_t* out) {
  const auto& d = static_cast<op::Ast*>(a)->shape.dims();
  for (size_t i = 0; i < d.size(); ++i) out[i] = d[i];
}
int ugh_op_ast_dtype(void* a) { return (int)static_cast<op::Ast*>(a)->dtype; }
// ug-pyo3/src/lib.rs:230-237
int ugh_op_store(void* arg, const size_t* dims, size_t rank, void* value, void** out) {
  return guard([&] {
    op::Store st;
    st.dst = static_cast<Arg*>(arg)->id;
    st.layout = Layout::from_shape(shape_of(dims, rank));
    st.value = *static_cast<op::Ast*>(value);
    *out = new op::Store(std::move(st));
  });
}
void ugh_op_store_free(void* s) { delete static_cast<op::Store*>(s); }
// ug-pyo3/src/lib.rs:244-265
int ugh_op_kernel_new(const char* name, void** args, size_t n_args, void** stores, size_t n_stores, void** out) {
  return guard([&] {
    op::Kernel k;
    k.name = name ? name : "";
    for (size_t i = 0; i < n_args; ++i) k.args.push_back(*static_cast<Arg*>(args[i]));
    for (size_t i = 0; i < n_stores; ++i) k.ops.push_back(*static_cast<op::Store*>(stores[i]));
    *out = new op::Kernel(std::move(k));
  });
}
void ugh_op_kernel_free(void* k) { delete static_cast<op::Kernel*>(k); }
int ugh_op_kernel_lower(void* k, void** out) {
  return guard([&] { *out = new ssa::Kernel(static_cast<op::Kernel*>(k)->lower(op::Opts{})); });
}
size_t ugh_op_kernel_str(void* k, char* buf, size_t buf_len) {
  const op::Kernel& kk = *static_cast<op::Kernel*>(k);
  std::string s = "Kernel { name: \"" + kk.name + "\", args: [";
  for (size_t i = 0; i < kk.args.size(); ++i) s += (i ? ", " : "") + std::to_string(kk.args[i].id.v);
  s += "], ops: [";
  for (size_t i = 0; i < kk.ops.size(); ++i)
    s += std::string(i ? ", " : "") + "Store { dst: " + std::to_string(kk.ops[i].dst.v) + ", shape: " + kk.ops[i].layout.shape().str() + ", value: " + ast_str(kk.ops[i].value) + " }";
  return copy_out(s + "] }", buf, buf_len);
}
size_t ugh_ssa_str(void* kernel, char* buf, size_t buf_len) { return copy_out(ssa_str(*static_cast<ssa::Kernel*>(kernel)), buf, buf_len); }
int ugh_ssa_flops_mem(void* kernel, size_t* flops, size_t* mem) {
  return guard([&] { flops_mem(*static_cast<ssa::Kernel*>(kernel), flops, mem); });
}
// Device::compile_cu as ug-pyo3 exposes it (ug-pyo3/src/lib.rs:438-456), for HIP source text.
int ugh_hip_compile_source(void* d, const char* source, const char* entry, size_t n_args, const int* arg_dtypes, uint32_t grid, uint32_t block,
                           uint32_t shared, void** out) {
  return guard([&] {
    HipDevice* hd = dynamic_cast<HipDevice*>(dev_of(d).get());
    if (!hd) bail("compile_hip needs the HIP device");
    ughip_func* f = nullptr;
    if (ughip_compile_source(hd->raw(), source, entry, n_args, arg_dtypes, grid, block, shared, &f)) bail(ughip_last_error());
    *out = new std::shared_ptr<Func>(std::make_shared<HipFunc>(f));
  });
}

// ---- lazy buffers ---------------------------------------------------------------------------------
int ugh_lb_cst(void* d, int dtype, double v, const size_t* dims, size_t rank, void** out) {
  return guard([&] { *out = box(LazyBuffer::cst(const_of(dtype, v), shape_of(dims, rank), dev_of(d))); });
}
int ugh_lb_copy(void* d, int dtype, const void* data, size_t len, const size_t* dims, size_t rank, void** out) {
  return guard([&] { *out = box(LazyBuffer::copy(data, (DType)dtype, len, shape_of(dims, rank), dev_of(d))); });
}
int ugh_lb_alloc_uninit(void* d, int dtype, const size_t* dims, size_t rank, void** out) {
  return guard([&] { *out = box(LazyBuffer::alloc_uninit((DType)dtype, shape_of(dims, rank), dev_of(d))); });
}
void ugh_lb_free(void* lb) { delete static_cast<LazyBuffer*>(lb); }
int ugh_lb_unary(void* lb, int op, void** out) {
  return guard([&] { *out = box(lb_of(lb).unary((UnaryOp)op)); });
}
int ugh_lb_cast(void* lb, int dtype, void** out) {
  return guard([&] { *out = box(lb_of(lb).cast((DType)dtype)); });
}
int ugh_lb_binary(void* lb, int op, void* rhs, void** out) {
  return guard([&] { *out = box(lb_of(lb).binary((BinaryOp)op, lb_of(rhs))); });
}
int ugh_lb_reduce(void* lb, int op, long dim, void** out) {
  return guard([&] { *out = box(lb_of(lb).reduce((ReduceOp)op, dim)); });
}
int ugh_lb_matmul(void* lb, void* rhs, int transpose, void** out) {
  return guard([&] { *out = box(lb_of(lb).matmul_(lb_of(rhs), transpose != 0)); });
}
int ugh_lb_split_dim(void* lb, long dim, size_t s1, size_t s2, void** out) {
  return guard([&] { *out = box(lb_of(lb).split_dim(dim, s1, s2)); });
}
int ugh_lb_merge_dims(void* lb, long dim, void** out) {
  return guard([&] { *out = box(lb_of(lb).merge_dims(dim)); });
}
int ugh_lb_squeeze(void* lb, long dim, void** out) {
  return guard([&] { *out = box(lb_of(lb).squeeze(dim)); });
}
int ugh_lb_unsqueeze(void* lb, long dim, void** out) {
  return guard([&] { *out = box(lb_of(lb).unsqueeze(dim)); });
}
int ugh_lb_get_on_dim(void* lb, long dim, size_t index, void** out) {
  return guard([&] { *out = box(lb_of(lb).get_on_dim(dim, index)); });
}
int ugh_lb_reshape(void* lb, const size_t* dims, size_t rank, void** out) {
  return guard([&] { *out = box(lb_of(lb).reshape(shape_of(dims, rank))); });
}
int ugh_lb_narrow(void* lb, long dim, size_t offset, size_t length, void** out) {
  return guard([&] { *out = box(lb_of(lb).narrow(dim, offset, length)); });
}
int ugh_lb_broadcast(void* lb, const size_t* dims, size_t rank, void** out) {
  return guard([&] { *out = box(lb_of(lb).broadcast(shape_of(dims, rank))); });
}
int ugh_lb_transpose(void* lb, long d1, long d2, void** out) {
  return guard([&] { *out = box(lb_of(lb).transpose(d1, d2)); });
}
int ugh_lb_cat(void** lbs, size_t n, long dim, void** out) {
  return guard([&] {
    std::vector<LazyBuffer> v;
    for (size_t i = 0; i < n; ++i) v.push_back(lb_of(lbs[i]));
    *out = box(LazyBuffer::cat(v, dim));
  });
}
int ugh_lb_set(void* lb, void* values, void** out) {
  return guard([&] { *out = box(lb_of(lb).set(lb_of(values))); });
}
int ugh_lb_set_l(void* lb, void* values, const size_t* dims, const size_t* strides, size_t rank, size_t offset, void** out) {
  return guard([&] {
    Layout l;
    l.shape_ = shape_of(dims, rank);
    l.strides_.assign(strides, strides + rank);
    l.offset_ = offset;
    *out = box(lb_of(lb).set_l(lb_of(values), l));
  });
}
int ugh_lb_custom(void* d, ugh_custom_fn fn, void* user, void** args, size_t n, const size_t* dims, size_t rank, int dtype, void** out) {
  return guard([&] {
    std::vector<LazyBuffer> v;
    for (size_t i = 0; i < n; ++i) v.push_back(lb_of(args[i]));
    *out = box(LazyBuffer::custom(wrap_cb(fn, user), v, shape_of(dims, rank), (DType)dtype, dev_of(d)));
  });
}
int ugh_lb_custom_ip(void* lb, ugh_custom_fn fn, void* user, void** args, size_t n, void** out) {
  return guard([&] {
    std::vector<LazyBuffer> v;
    for (size_t i = 0; i < n; ++i) v.push_back(lb_of(args[i]));
    *out = box(lb_of(lb).custom_ip(wrap_cb(fn, user), v));
  });
}
int ugh_lb_ssa(void* d, void* kernel, void** args, size_t n, const size_t* dims, size_t rank, int dtype, void** out) {
  return guard([&] {
    std::vector<LazyBuffer> v;
    for (size_t i = 0; i < n; ++i) v.push_back(lb_of(args[i]));
    *out = box(LazyBuffer::ssa(*static_cast<ssa::Kernel*>(kernel), v, shape_of(dims, rank), (DType)dtype, dev_of(d)));
  });
}
size_t ugh_lb_rank(void* lb) { return static_cast<LazyBuffer*>(lb)->rank(); }
void ugh_lb_dims(void* lb, size_t* out) {
  const auto& d = static_cast<LazyBuffer*>(lb)->dims();
  std::memcpy(out, d.data(), d.size() * sizeof(size_t));
}
int ugh_lb_dtype(void* lb) { return (int)static_cast<LazyBuffer*>(lb)->dtype(); }
size_t ugh_lb_elem_count(void* lb) { return static_cast<LazyBuffer*>(lb)->elem_count(); }
int ugh_lb_realized(void* lb) { return static_cast<LazyBuffer*>(lb)->realized(); }
int ugh_lb_realize(void* lb) {
  return guard([&] { lb_of(lb).realize(); });
}
int ugh_lb_data_vec(void* lb, int dtype, void* out, size_t len) {
  return guard([&] {
    if (len != lb_of(lb).elem_count()) bail("data_vec: output length mismatch");
    lb_of(lb).data_vec(out, (DType)dtype);
  });
}
// Overwrite the realised storage behind `lb` (the tests that poke at `lb.data()` in lb_tests.rs:82-94).
int ugh_lb_write(void* lb, const void* data, int dtype, size_t len) {
  return guard([&] {
    LazyBuffer& b = lb_of(lb);
    if (!b.data()->slice) bail("no data");
    b.data()->slice->copy_host_to_device(data, (DType)dtype, len);
  });
}

// ---- schedules ----------------------------------------------------------------------------------------
int ugh_schedule_create(void** lbs, size_t n, void** out) {
  return guard([&] {
    std::vector<LazyBuffer> v;
    for (size_t i = 0; i < n; ++i) v.push_back(lb_of(lbs[i]));
    *out = new Schedule(Schedule::create(v));
  });
}
void ugh_schedule_free(void* s) { delete static_cast<Schedule*>(s); }
size_t ugh_schedule_n_items(void* s) { return static_cast<Schedule*>(s)->items().size(); }
int ugh_schedule_item_kind(void* s, size_t i) { return (int)static_cast<Schedule*>(s)->items().at(i).kind; }
size_t ugh_schedule_item_n_args(void* s, size_t i) {
  const ScheduleItem& it = static_cast<Schedule*>(s)->items().at(i);
  return it.kind == ScheduleItem::Kernel ? it.kernel.args.size() : it.args.size();
}
// Kernel items only: name (lower_op.rs:561-633) and the SSA from `optimize().lower(Opts::default())`.
int ugh_schedule_item_name(void* s, size_t i, char* buf, size_t buf_len) {
  return guard([&] {
    const ScheduleItem& it = static_cast<Schedule*>(s)->items().at(i);
    if (it.kind != ScheduleItem::Kernel) bail("not a kernel item");
    std::string n = it.kernel.kernel().ops[0].name();
    snprintf(buf, buf_len, "%s", n.c_str());
  });
}
int ugh_schedule_item_ssa(void* s, size_t i, int optimize, void** out) {
  return guard([&] {
    const ScheduleItem& it = static_cast<Schedule*>(s)->items().at(i);
    if (it.kind == ScheduleItem::Ssa) {
      *out = new ssa::Kernel(it.ssa);
      return;
    }
    if (it.kind != ScheduleItem::Kernel) bail("not a kernel item");
    op::Kernel k = it.kernel.kernel();
    if (optimize) k = k.optimize();
    *out = new ssa::Kernel(k.lower(op::Opts()));
  });
}
void* ugh_cache_new(void) { return new CompilationCache(); }
void ugh_cache_free(void* c) { delete static_cast<CompilationCache*>(c); }
size_t ugh_cache_size(void* c) {
  CompilationCache* cc = static_cast<CompilationCache*>(c);
  return cc->op_cache.size() + cc->ssa_cache.size();
}
int ugh_schedule_compile(void* s, void* cache, void** out) {
  return guard([&] {
    Schedule* sc = static_cast<Schedule*>(s);
    CompiledBox* b = new CompiledBox();
    try {
      if (cache) b->cs = sc->compile_with_cache(*static_cast<CompilationCache*>(cache));
      else b->cs = sc->compile();
    } catch (...) {
      delete b;
      throw;
    }
    *out = b;
  });
}
void ugh_compiled_free(void* c) { delete static_cast<CompiledBox*>(c); }
int ugh_compiled_run(void* c) {
  return guard([&] { static_cast<CompiledBox*>(c)->cs.run(); });
}
size_t ugh_compiled_n_funcs(void* c) { return static_cast<CompiledBox*>(c)->cs.funcs.size(); }
int ugh_compiled_func_kind(void* c, size_t i) { return (int)static_cast<CompiledBox*>(c)->cs.funcs.at(i).kind; }
void* ugh_compiled_func_raw_hip(void* c, size_t i) {
  const CompiledFunc& f = static_cast<CompiledBox*>(c)->cs.funcs.at(i);
  HipFunc* h = f.func ? dynamic_cast<HipFunc*>(f.func.get()) : nullptr;
  return h ? h->raw() : nullptr;
}

// ---- safetensors (ug-core/src/safetensors.rs) ---------------------------------------------------------
int ugh_safetensors_open(const char* const* paths, size_t n_paths, void** out) {
  return guard([&] {
    if (n_paths == 0) bail("no safetensors file given");
    if (n_paths == 1) {
      *out = new ug::MmapedSafetensors(ug::MmapedSafetensors::open(paths[0]));
    } else {
      std::vector<std::string> ps(paths, paths + n_paths);
      *out = new ug::MmapedSafetensors(ug::MmapedSafetensors::multi(ps));
    }
  });
}
void ugh_safetensors_free(void* h) { delete static_cast<ug::MmapedSafetensors*>(h); }
size_t ugh_safetensors_count(void* h) { return static_cast<ug::MmapedSafetensors*>(h)->tensors().size(); }
// Entry i in file/header order: name and dtype as NUL-terminated strings, up to 8 dims.
int ugh_safetensors_entry(void* h, size_t i, char* name, size_t name_cap, char* dtype, size_t dtype_cap, size_t* rank, size_t* dims, size_t* nbytes) {
  return guard([&] {
    auto ts = static_cast<ug::MmapedSafetensors*>(h)->tensors();
    if (i >= ts.size()) bail("entry index out of range");
    snprintf(name, name_cap, "%s", ts[i].first.c_str());
    snprintf(dtype, dtype_cap, "%s", ts[i].second.dtype.c_str());
    if (ts[i].second.shape.size() > 8) bail("more than 8 dims");
    *rank = ts[i].second.shape.size();
    for (size_t k = 0; k < ts[i].second.shape.size(); ++k) dims[k] = ts[i].second.shape[k];
    *nbytes = ts[i].second.nbytes;
  });
}
// cast_dtype < 0: load in the stored dtype (safetensors.rs:71-74), else load_with_cast (:76-84).
int ugh_safetensors_load(void* h, const char* name, void* device, int cast_dtype, void** out_lb, int* cast_on_device) {
  return guard([&] {
    auto& st = *static_cast<ug::MmapedSafetensors*>(h);
    if (cast_dtype < 0) {
      *out_lb = box(st.load(name, dev_of(device)));
      if (cast_on_device) *cast_on_device = 0;
    } else {
      *out_lb = box(st.load_with_cast(name, (DType)cast_dtype, dev_of(device)));
      if (cast_on_device) *cast_on_device = st.last_cast_on_device() ? 1 : 0;
    }
  });
}

// ---- ug-llama ---------------------------------------------------------------------------------------------
using OpsPtr = std::shared_ptr<ug_llama::Ops>;
int ugh_llama_ops_hip(void** out) {
  return guard([&] { *out = new OpsPtr(ug_llama::hip_ops()); });
}
int ugh_llama_ops_hip_ex(int bf16x3, void** out) {
  return guard([&] { *out = new OpsPtr(ug_llama::hip_ops(bf16x3 != 0)); });
}
void ugh_llama_ops_free(void* o) { delete static_cast<OpsPtr*>(o); }
static ug_llama::Ops& ops_of(void* o) {
  if (!o) bail("null ops");
  return **static_cast<OpsPtr*>(o);
}
int ugh_llama_rope(void* ops, void* src, void* cos, void* sin, void* pos, int interleaved, void** out) {
  return guard([&] {
    *out = box(interleaved ? ops_of(ops).rope_i(lb_of(src), lb_of(cos), lb_of(sin), lb_of(pos))
                           : ops_of(ops).rope(lb_of(src), lb_of(cos), lb_of(sin), lb_of(pos)));
  });
}
int ugh_llama_cat(void* ops, void* lhs, void* rhs, size_t axis, void** out) {
  return guard([&] { *out = box(ops_of(ops).cat(lb_of(lhs), lb_of(rhs), axis)); });
}
int ugh_llama_custom_softmax(void* ops, void* src, void** out) {
  return guard([&] { *out = box(ops_of(ops).custom_softmax(lb_of(src))); });
}
int ugh_llama_causal_mask(void* ops, void* src, void** out) {
  return guard([&] { *out = box(ops_of(ops).causal_mask(lb_of(src))); });
}
int ugh_llama_causal_softmax(void* ops, void* src, void** out) {
  return guard([&] { *out = box(ops_of(ops).causal_softmax(lb_of(src))); });
}
int ugh_llama_attention_decode(void* ops, void* q, void* k, void* v, float scale, void** out) {
  return guard([&] { *out = box(ops_of(ops).attention_decode(lb_of(q), lb_of(k), lb_of(v), scale)); });
}
int ugh_llama_rope_append(void* ops, void* cache, void* x, void* cos, void* sin, void* pos, int interleaved, void** out) {
  return guard([&] {
    if (cos) *out = box(ops_of(ops).rope_append(lb_of(cache), lb_of(x), &lb_of(cos), &lb_of(sin), &lb_of(pos), interleaved != 0));
    else *out = box(ops_of(ops).rope_append(lb_of(cache), lb_of(x), nullptr, nullptr, nullptr, false));
  });
}
int ugh_llama_attention_decode_flat(void* ops, void* q, void* k, void* v, float scale, void* cos, void* sin, void* pos, int interleaved, void** out) {
  return guard([&] {
    if (cos) *out = box(ops_of(ops).attention_decode_flat(lb_of(q), lb_of(k), lb_of(v), scale, &lb_of(cos), &lb_of(sin), &lb_of(pos), interleaved != 0));
    else *out = box(ops_of(ops).attention_decode_flat(lb_of(q), lb_of(k), lb_of(v), scale, nullptr, nullptr, nullptr, false));
  });
}
int ugh_llama_kv_cache_capacity(void* ops, size_t max_positions, size_t head_dim, size_t* out) {
  return guard([&] { *out = ops_of(ops).kv_cache_capacity(max_positions, head_dim); });
}
int ugh_llama_kv_append(void* ops, void* cache, size_t len, void* x, void* cos, void* sin, void* pos, int interleaved, size_t x_offset, size_t x_row_stride,
                        void** out) {
  return guard([&] {
    if (cos) *out = box(ops_of(ops).kv_append(lb_of(cache), len, lb_of(x), &lb_of(cos), &lb_of(sin), &lb_of(pos), interleaved != 0, x_offset, x_row_stride));
    else *out = box(ops_of(ops).kv_append(lb_of(cache), len, lb_of(x), nullptr, nullptr, nullptr, false, x_offset, x_row_stride));
  });
}
int ugh_llama_attention_cached(void* ops, void* q, void* k, void* v, size_t s, float scale, void* cos, void* sin, void* pos, int interleaved, size_t q_offset,
                               size_t q_row_stride, size_t n_heads, void** out) {
  return guard([&] {
    if (cos)
      *out = box(ops_of(ops).attention_cached(lb_of(q), lb_of(k), lb_of(v), s, scale, &lb_of(cos), &lb_of(sin), &lb_of(pos), interleaved != 0, q_offset, q_row_stride,
                                              n_heads));
    else *out = box(ops_of(ops).attention_cached(lb_of(q), lb_of(k), lb_of(v), s, scale, nullptr, nullptr, nullptr, false, q_offset, q_row_stride, n_heads));
  });
}
int ugh_llama_attention_step(void* ops, void* qkv, void* kcache, void* vcache, size_t len, size_t n_heads, float scale, void* cos, void* sin, void* pos,
                             int interleaved, void** out) {
  return guard([&] {
    if (cos) *out = box(ops_of(ops).attention_step(lb_of(qkv), lb_of(kcache), lb_of(vcache), len, n_heads, scale, &lb_of(cos), &lb_of(sin), &lb_of(pos), interleaved != 0));
    else *out = box(ops_of(ops).attention_step(lb_of(qkv), lb_of(kcache), lb_of(vcache), len, n_heads, scale, nullptr, nullptr, nullptr, false));
  });
}
int ugh_llama_attention_steps(void* ops, void* qkv, void* kcache, void* vcache, size_t len, size_t n_heads, float scale, void* cos, void* sin, void* pos,
                              int interleaved, void** out) {
  return guard([&] {
    if (cos) *out = box(ops_of(ops).attention_steps(lb_of(qkv), lb_of(kcache), lb_of(vcache), len, n_heads, scale, &lb_of(cos), &lb_of(sin), &lb_of(pos), interleaved != 0));
    else *out = box(ops_of(ops).attention_steps(lb_of(qkv), lb_of(kcache), lb_of(vcache), len, n_heads, scale, nullptr, nullptr, nullptr, false));
  });
}
int ugh_llama_attention_steps_add(void* ops, void* qkv, void* kcache, void* vcache, size_t len, size_t n_heads, float scale, void* cos, void* sin, void* pos,
                                  int interleaved, void* w_o, void* residual, void** out) {
  return guard([&] {
    *out = box(ops_of(ops).attention_steps_add(lb_of(qkv), lb_of(kcache), lb_of(vcache), len, n_heads, scale, cos ? &lb_of(cos) : nullptr, cos ? &lb_of(sin) : nullptr,
                                               cos ? &lb_of(pos) : nullptr, cos && interleaved != 0, lb_of(w_o), lb_of(residual)));
  });
}
int ugh_llama_linear_norm(void* ops, void* x, void* alpha, float eps, void* w, void** out) {
  return guard([&] { *out = box(ops_of(ops).linear_norm(lb_of(x), lb_of(alpha), eps, lb_of(w))); });
}
int ugh_llama_mlp_stacked(void* ops, void* x, void* alpha, float eps, void* w_gate_up, void* w_down, void* residual, void** out) {
  return guard([&] { *out = box(ops_of(ops).mlp_stacked(lb_of(x), alpha ? &lb_of(alpha) : nullptr, eps, lb_of(w_gate_up), lb_of(w_down), lb_of(residual))); });
}
int ugh_llama_device_argmax(void* ops) { return ops_of(ops).device_argmax() ? 1 : 0; }
int ugh_llama_argmax_into(void* ops, void* token, void* logits, size_t row, void* ids, void* vals, size_t slot, void** out) {
  return guard([&] { *out = box(ops_of(ops).argmax_into(lb_of(token), lb_of(logits), row, lb_of(ids), lb_of(vals), slot)); });
}
int ugh_llama_packed_projections(void* ops) { return ops_of(ops).packed_projections() ? 1 : 0; }
int ugh_llama_linear_packed(void* ops, void* x, size_t n_mats, void** ws, void* alpha, float eps, void** out) {
  return guard([&] {
    std::vector<ug::LazyBuffer> w;
    for (size_t i = 0; i < n_mats; ++i) w.push_back(lb_of(ws[i]));
    *out = box(ops_of(ops).linear_packed(lb_of(x), w, alpha ? &lb_of(alpha) : nullptr, eps));
  });
}
int ugh_llama_gate_up(void* ops, void* x, void* w_gate, void* w_up, void* alpha, float eps, void** out) {
  return guard([&] { *out = box(ops_of(ops).gate_up(lb_of(x), lb_of(w_gate), lb_of(w_up), alpha ? &lb_of(alpha) : nullptr, eps)); });
}
int ugh_llama_gate_up_stacked(void* ops, void* x, void* w, void** out) {
  return guard([&] { *out = box(ops_of(ops).gate_up_stacked(lb_of(x), lb_of(w))); });
}
int ugh_llama_linear(void* ops, void* x, void* w, void** out) {
  return guard([&] { *out = box(ops_of(ops).linear(*static_cast<LazyBuffer*>(x), *static_cast<LazyBuffer*>(w))); });
}
int ugh_llama_linear_add(void* ops, void* x, void* w, void* residual, void** out) {
  return guard([&] { *out = box(ops_of(ops).linear_add(lb_of(x), lb_of(w), lb_of(residual))); });
}
int ugh_llama_rms_norm(void* src, void* alpha, float eps, void** out) {
  return guard([&] { *out = box(ug_llama::rms_norm(lb_of(src), lb_of(alpha), eps)); });
}
int ugh_llama_softmax(void* src, void** out) {
  return guard([&] { *out = box(ug_llama::softmax(lb_of(src))); });
}
int ugh_llama_silu(void* src, void** out) {
  return guard([&] { *out = box(ug_llama::silu(lb_of(src))); });
}
int ugh_llama_repeat(void* src, size_t axis, size_t n_rep, void** out) {
  return guard([&] { *out = box(ug_llama::repeat(lb_of(src), axis, n_rep)); });
}
int ugh_llama_index_select(void* src, void* ids, void** out) {
  return guard([&] { *out = box(ug_llama::index_select(lb_of(src), lb_of(ids))); });
}
static ug_llama::Config cfg_of(const ugh_llama_config* c) {
  ug_llama::Config cfg;
  cfg.hidden_size = c->hidden_size;
  cfg.intermediate_size = c->intermediate_size;
  cfg.max_position_embeddings = c->max_position_embeddings;
  cfg.num_attention_heads = c->num_attention_heads;
  cfg.num_key_value_heads = c->num_key_value_heads;
  cfg.num_hidden_layers = c->num_hidden_layers;
  cfg.rms_norm_eps = c->rms_norm_eps;
  cfg.rope_interleaved = c->rope_interleaved != 0;
  cfg.rope_theta = c->rope_theta;
  cfg.vocab_size = c->vocab_size;
  return cfg;
}
int ugh_llama_rope_tables(void* d, const ugh_llama_config* c, void** cos, void** sin) {
  return guard([&] {
    ug_llama::Rope r = ug_llama::Rope::create(cfg_of(c), dev_of(d));
    *cos = box(r.cos);
    *sin = box(r.sin);
  });
}
int ugh_llama_model_new(void* d, void* ops, const ugh_llama_config* c, int custom_softmax, uint64_t seed, float std, int round_bf16, void** out) {
  return guard([&] {
    auto w = ug_llama::synthetic_weights(seed, std, round_bf16 != 0);
    *out = new ug_llama::Model(cfg_of(c), custom_softmax != 0, *w, dev_of(d), *static_cast<OpsPtr*>(ops));
  });
}
int ugh_llama_model_new_ex(void* d, void* ops, const ugh_llama_config* c, int custom_softmax, uint64_t seed, float std, int round_bf16, float norm_mean, float embed_std,
                           void** out) {
  return guard([&] {
    auto w = ug_llama::synthetic_weights(seed, std, round_bf16 != 0, norm_mean, embed_std);
    *out = new ug_llama::Model(cfg_of(c), custom_softmax != 0, *w, dev_of(d), *static_cast<OpsPtr*>(ops));
  });
}
int ugh_llama_model_from_safetensors(void* d, void* ops, const ugh_llama_config* c, int custom_softmax, const char* const* paths, size_t n_paths, void** out) {
  return guard([&] {
    std::vector<std::string> ps(paths, paths + n_paths);
    auto w = ug_llama::safetensors_weights(ps);
    *out = new ug_llama::Model(cfg_of(c), custom_softmax != 0, *w, dev_of(d), *static_cast<OpsPtr*>(ops));
  });
}
void ugh_llama_model_free(void* m) { delete static_cast<ug_llama::Model*>(m); }
int ugh_llama_model_set_fused_attention(void* m, int on) {
  return guard([&] { static_cast<ug_llama::Model*>(m)->set_fused_attention(on); });
}
int ugh_llama_model_store_matrices_bf16(void* m) {
  return guard([&] { static_cast<ug_llama::Model*>(m)->store_matrices_bf16(); });
}
int ugh_llama_generate(void* m, const int32_t* prompt, size_t n_prompt, size_t n_steps, int32_t* out_tokens, double* prefill_ms,
                       double* decode_ms, float* margins) {
  return guard([&] {
    ug_llama::GenerateStats st;
    std::vector<int32_t> p(prompt, prompt + n_prompt);
    std::vector<int32_t> toks = ug_llama::generate_greedy(*static_cast<ug_llama::Model*>(m), p, n_steps, &st);
    std::memcpy(out_tokens, toks.data(), toks.size() * sizeof(int32_t));
    if (prefill_ms) *prefill_ms = st.prefill_ms;
    if (decode_ms) *decode_ms = st.decode_ms;
    if (margins) std::memcpy(margins, st.top1_margin.data(), st.top1_margin.size() * sizeof(float));
  });
}
int ugh_llama_set_switch(const char* name, int on) {
  return guard([&] {
    if (!name || !ug_llama::set_switch(name, on != 0)) throw std::runtime_error(std::string("no llama switch named '") + (name ? name : "(null)") + "'");
  });
}
static thread_local size_t g_last_decode_items = 0;
int ugh_llama_generate_ex(void* m, const int32_t* prompt, size_t n_prompt, size_t n_steps, const int32_t* forced, int32_t* out_tokens, double* prefill_ms,
                          double* decode_ms, float* margins, float* top1_values) {
  return guard([&] {
    ug_llama::GenerateStats st;
    std::vector<int32_t> p(prompt, prompt + n_prompt), f;
    if (forced) f.assign(forced, forced + n_steps);
    std::vector<int32_t> toks = ug_llama::generate_greedy(*static_cast<ug_llama::Model*>(m), p, n_steps, &st, forced ? &f : nullptr);
    std::memcpy(out_tokens, toks.data(), toks.size() * sizeof(int32_t));
    if (prefill_ms) *prefill_ms = st.prefill_ms;
    if (decode_ms) *decode_ms = st.decode_ms;
    if (margins) std::memcpy(margins, st.top1_margin.data(), st.top1_margin.size() * sizeof(float));
    if (top1_values) std::memcpy(top1_values, st.top1_value.data(), st.top1_value.size() * sizeof(float));
    g_last_decode_items = st.decode_items;
  });
}
// Schedule items (device launches) of the last single-token step of this thread's last ugh_llama_generate_ex.
size_t ugh_llama_last_decode_items() { return g_last_decode_items; }
int ugh_synthetic_weights(uint64_t seed, float std, int round_bf16, const char* name, size_t n, float* out) {
  return guard([&] {
    auto w = ug_llama::synthetic_weights(seed, std, round_bf16 != 0);
    std::vector<float> v = w->get(name, {n});
    std::memcpy(out, v.data(), n * sizeof(float));
  });
}

}  // extern "C"
