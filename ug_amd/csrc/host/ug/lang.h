// The two IRs on the path: `op` (tensor-level AST) and `ssa` (flat kernel IR).
// Mirrors ug-core/src/lang.rs:408-823.  ssa instructions are stored directly in the wire
// format of include/ughip.h, so handing a kernel to the backend is a pointer, not a copy.
#pragma once
#include <atomic>
#include <cstring>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "core.h"

namespace ug {

// lang.rs:82-102: process-wide unique argument ids.
struct ArgId {
  size_t v = 0;
  static ArgId fresh() {
    static std::atomic<size_t> counter{1};
    return ArgId{counter.fetch_add(1)};
  }
  bool operator<(const ArgId& o) const { return v < o.v; }
  bool operator==(const ArgId& o) const { return v == o.v; }
};

// lang.rs:138-178 (only pointer arguments exist on this path).
struct Arg {
  ArgId id;
  DType dtype = DType::F32;
  bool is_ptr = true;
  static Arg ptr(DType d) { return Arg{ArgId::fresh(), d, true}; }
};

namespace ssa {

using A = ughip_a;
using Instr = ughip_instr;

inline A var(uint32_t v) {
  A a{};
  a.var = v;
  return a;
}
inline A cst(const Const& c) {
  A a{};
  a.is_const = 1;
  a.dtype = (uint8_t)c.dtype;
  a.i = c.i;
  a.f = c.f;
  return a;
}
inline A i32(int32_t v) { return cst(Const::i32(v)); }

inline Instr mk(int op, DType dt = DType::F32, int sub = 0, uint32_t v = 0, uint64_t n = 0, A a = A{}, A b = A{}) {
  Instr i{};
  i.op = op;
  i.dtype = (int)dt;
  i.sub = sub;
  i.v = v;
  i.n = n;
  i.a = a;
  i.b = b;
  return i;
}
inline Instr define_acc(const Const& c) { return mk(UGHIP_I_DEFINE_ACC, c.dtype, 0, 0, 0, cst(c)); }
inline Instr define_global(size_t index, DType dt) { return mk(UGHIP_I_DEFINE_GLOBAL, dt, 0, 0, index); }
inline Instr define_local(size_t size, DType dt) { return mk(UGHIP_I_DEFINE_LOCAL, dt, 0, 0, size); }
inline Instr special(int which) { return mk(UGHIP_I_SPECIAL, DType::I32, which); }
inline Instr constant(const Const& c) { return mk(UGHIP_I_CONST, c.dtype, 0, 0, 0, cst(c)); }
inline Instr unary(UnaryOp op, A arg, DType dt) { return mk(UGHIP_I_UNARY, dt, (int)op, 0, 0, arg); }
inline Instr binary(BinaryOp op, A lhs, A rhs, DType dt) { return mk(UGHIP_I_BINARY, dt, (int)op, 0, 0, lhs, rhs); }
inline Instr range(A lo, A up, size_t step, uint32_t end_idx) { return mk(UGHIP_I_RANGE, DType::I32, 0, end_idx, step, lo, up); }
inline Instr load(uint32_t src, A offset, DType dt) { return mk(UGHIP_I_LOAD, dt, 0, src, 0, offset); }
inline Instr assign(uint32_t dst, A src) { return mk(UGHIP_I_ASSIGN, DType::F32, 0, dst, 0, src); }
inline Instr end_range(uint32_t start_idx) { return mk(UGHIP_I_END_RANGE, DType::F32, 0, start_idx); }
inline Instr if_(A cond, uint32_t end_idx) { return mk(UGHIP_I_IF, DType::F32, 0, end_idx, 0, cond); }
inline Instr end_if() { return mk(UGHIP_I_END_IF); }
inline Instr store(uint32_t dst, A offset, A value, DType dt) { return mk(UGHIP_I_STORE, dt, 0, dst, 0, offset, value); }
inline Instr barrier() { return mk(UGHIP_I_BARRIER); }
inline Instr reduce_local(ReduceOp op, A arg, DType dt) { return mk(UGHIP_I_REDUCE_LOCAL, dt, (int)op, 0, 0, arg); }

// ssa::Kernel (lang.rs:711-753)
struct Kernel {
  std::vector<Instr> instrs;
  std::vector<ughip_kernel_arg> args;
  LaunchConfig launch_config;

  Kernel() = default;
  Kernel(std::vector<Instr> i, std::vector<ughip_kernel_arg> a, LaunchConfig c) : instrs(std::move(i)), args(std::move(a)), launch_config(c) {}

  // lang.rs:739-753: arguments are the DefineGlobal lines, in order; grid 1 x block 1.
  static Kernel from_instrs(std::vector<Instr> instrs) {
    std::vector<ughip_kernel_arg> args;
    for (size_t line = 0; line < instrs.size(); ++line) {
      const Instr& in = instrs[line];
      if (in.op != UGHIP_I_DEFINE_GLOBAL) continue;
      if (in.n != args.size()) bail("unexpected order for arguments in kernel");
      ughip_kernel_arg a{};
      a.arg_id = ArgId::fresh().v;
      a.is_ptr = 1;
      a.dtype = (uint8_t)in.dtype;
      a.var = (uint32_t)line;
      args.push_back(a);
    }
    return Kernel(std::move(instrs), std::move(args), LaunchConfig{1, 1, 0});
  }

  ughip_ssa wire() const {
    ughip_ssa s{};
    s.instrs = instrs.data();
    s.n_instrs = instrs.size();
    s.args = args.data();
    s.n_args = args.size();
    s.grid_dim = launch_config.grid_dim;
    s.block_dim = launch_config.block_dim;
    s.shared_mem = launch_config.shared_mem;
    return s;
  }

  // Byte image of the instruction list: the key of CompilationCache::ssa_cache (cache.rs:6,76).
  std::string instrs_key() const { return std::string(reinterpret_cast<const char*>(instrs.data()), instrs.size() * sizeof(Instr)); }
};

}  // namespace ssa

namespace op {

// lang.rs:422-429
struct LayoutOp {
  enum Kind { Broadcast, Narrow, Transpose, SplitDim, MergeDims } kind = Broadcast;
  size_t inserted_dims = 0;
  std::vector<size_t> broadcasted_dims;
  size_t dim = 0, offset = 0;   // Narrow; SplitDim/MergeDims use dim
  size_t dim1 = 0, dim2 = 0;    // Transpose
  size_t lhs = 0, rhs = 0;      // SplitDim / MergeDims
  std::string key() const {
    std::string s = "l" + std::to_string((int)kind) + ":" + std::to_string(inserted_dims) + ":";
    for (size_t d : broadcasted_dims) s += std::to_string(d) + ",";
    return s + ":" + std::to_string(dim) + ":" + std::to_string(offset) + ":" + std::to_string(dim1) + ":" + std::to_string(dim2) + ":" +
           std::to_string(lhs) + ":" + std::to_string(rhs);
  }
};

struct AstInner;
// lang.rs:415-420
struct Ast {
  std::shared_ptr<const AstInner> inner;
  DType dtype = DType::F32;
  Shape shape;
};

// lang.rs:431-444
struct AstInner {
  enum Kind { Id, Load, Reduce, Unary, Binary, Const, Layout } kind = Const;
  uint32_t id_src = 0;       // Id
  ArgId load_src;            // Load
  ug::Layout load_layout;    // Load
  ReduceOp reduce_op = ReduceOp::Sum;
  size_t reduce_dim = 0;
  UnaryOp unary_op = UnaryOp::Id;
  DType cast_to = DType::F32;  // Unary Cast
  BinaryOp binary_op = BinaryOp::Add;
  ug::Const cst;
  LayoutOp layout_op;
  Ast arg, rhs;  // arg doubles as the lhs of Binary
};

inline Ast make(AstInner in, DType dtype, Shape shape) { return Ast{std::make_shared<const AstInner>(std::move(in)), dtype, std::move(shape)}; }

inline Ast load(ArgId src, const ug::Layout& layout, DType dtype) {
  AstInner in;
  in.kind = AstInner::Load;
  in.load_src = src;
  in.load_layout = layout;
  return make(std::move(in), dtype, layout.shape());
}

// lang.rs:452-477
inline Ast broadcast(const Ast& arg, const Shape& shape) {
  if (arg.shape.rank() > shape.rank()) bail("target shape " + shape.str() + " has less dimensions than original shape " + arg.shape.str());
  LayoutOp op;
  op.kind = LayoutOp::Broadcast;
  op.inserted_dims = shape.rank() - arg.shape.rank();
  for (size_t i = 0; i < op.inserted_dims; ++i) op.broadcasted_dims.push_back(i);
  for (size_t i = 0; i < arg.shape.rank(); ++i) {
    size_t dim_idx = i + op.inserted_dims;
    if (shape.dims()[dim_idx] != arg.shape.dims()[i]) {
      if (arg.shape.dims()[i] == 1) op.broadcasted_dims.push_back(dim_idx);
      else bail("cannot broadcast from " + arg.shape.str() + " to " + shape.str());
    }
  }
  AstInner in;
  in.kind = AstInner::Layout;
  in.layout_op = op;
  in.arg = arg;
  return make(std::move(in), arg.dtype, shape);
}

inline Ast layout(const LayoutOp& op, const Ast& arg, const Shape& shape) {
  AstInner in;
  in.kind = AstInner::Layout;
  in.layout_op = op;
  in.arg = arg;
  return make(std::move(in), arg.dtype, shape);
}

inline Ast unary(UnaryOp op, const Ast& arg, DType cast_to = DType::F32) {
  AstInner in;
  in.kind = AstInner::Unary;
  in.unary_op = op;
  in.cast_to = cast_to;
  in.arg = arg;
  return make(std::move(in), op == UnaryOp::Cast ? cast_to : arg.dtype, arg.shape);
}

// lang.rs:496-505: keepdim.
inline Ast reduce(ReduceOp op, const Ast& arg, size_t dim) {
  std::vector<size_t> dims = arg.shape.dims();
  if (dim >= dims.size()) bail("no dim " + std::to_string(dim) + " in shape " + arg.shape.str());
  dims[dim] = 1;
  AstInner in;
  in.kind = AstInner::Reduce;
  in.reduce_op = op;
  in.reduce_dim = dim;
  in.arg = arg;
  return make(std::move(in), arg.dtype, Shape(dims));
}

// lang.rs:507-520: the result takes the lhs shape; only scalars broadcast implicitly.
inline Ast binary(BinaryOp op, const Ast& lhs, const Ast& rhs) {
  if (lhs.dtype != rhs.dtype) bail(std::string("dtype mismatch in binary op, lhs: ") + dtype_str(lhs.dtype) + ", rhs: " + dtype_str(rhs.dtype));
  if (lhs.shape != rhs.shape && lhs.shape.rank() != 0 && rhs.shape.rank() != 0)
    bail("shape mismatch in binary op, lhs: " + lhs.shape.str() + ", rhs: " + rhs.shape.str());
  AstInner in;
  in.kind = AstInner::Binary;
  in.binary_op = op;
  in.arg = lhs;
  in.rhs = rhs;
  return make(std::move(in), lhs.dtype, lhs.shape);
}

inline Ast cst(const ug::Const& c) {
  AstInner in;
  in.kind = AstInner::Const;
  in.cst = c;
  return make(std::move(in), c.dtype, Shape());
}

// lang.rs:522-527 (used by the `affine` test, basic_tests.rs:118-136).
inline Shape broadcast_shape_binary_op(const Shape& l, const Shape& r) {
  size_t rank = std::max(l.rank(), r.rank());
  std::vector<size_t> out(rank);
  for (size_t i = 0; i < rank; ++i) {
    size_t ld = i < rank - l.rank() ? 1 : l.dims()[i - (rank - l.rank())];
    size_t rd = i < rank - r.rank() ? 1 : r.dims()[i - (rank - r.rank())];
    if (ld != rd && ld != 1 && rd != 1) bail("shape mismatch in binary op, lhs: " + l.str() + ", rhs: " + r.str());
    out[i] = ld == 1 ? rd : ld;
  }
  return Shape(out);
}
inline Ast broadcast_binary(BinaryOp op, const Ast& lhs, const Ast& rhs) {
  Shape s = broadcast_shape_binary_op(lhs.shape, rhs.shape);
  return binary(op, broadcast(lhs, s), broadcast(rhs, s));
}

// lang.rs:550-569
inline void arg_ids(const Ast& ast, std::set<ArgId>& ids) {
  const AstInner& in = *ast.inner;
  switch (in.kind) {
    case AstInner::Layout:
    case AstInner::Reduce:
    case AstInner::Unary: arg_ids(in.arg, ids); break;
    case AstInner::Binary:
      arg_ids(in.arg, ids);
      arg_ids(in.rhs, ids);
      break;
    case AstInner::Load: ids.insert(in.load_src); break;
    default: break;
  }
}

// lang.rs:572-587
struct Store {
  ArgId dst;
  ug::Layout layout;
  Ast value;
  DType dtype() const { return value.dtype; }
  std::string name() const;        // lower_op.rs:561-633
  bool can_merge_all() const;      // lower_op.rs:636-664
};

struct Opts;

// lang.rs:589-604 + lower_op.rs:408-558
struct Kernel {
  std::string name;
  std::vector<Arg> args;
  std::vector<Store> ops;
  Kernel optimize() const;
  ssa::Kernel lower(const Opts& opts) const;
};

// lower_op.rs:6-44
struct ThreadBlock {
  size_t dim = 0, block_dim = 0;
};
struct Opts {
  bool has_thread_block = false, has_block_axis = false;
  ThreadBlock thread_block;
  size_t block_axis = 0;
  Opts with_global_axis(size_t axis, size_t block_dim) const {
    Opts o = *this;
    o.has_block_axis = true;
    o.block_axis = axis;
    o.has_thread_block = true;
    o.thread_block = {axis, block_dim};
    return o;
  }
  Opts with_block_axis(size_t axis) const {
    Opts o = *this;
    o.has_block_axis = true;
    o.block_axis = axis;
    return o;
  }
  Opts with_thread_block(size_t dim, size_t block_dim) const {
    Opts o = *this;
    o.has_thread_block = true;
    o.thread_block = {dim, block_dim};
    return o;
  }
};

// Structural key with argument ids replaced through `rename` (cache.rs:14-72).
std::string ast_key(const Ast& ast, const std::vector<std::pair<ArgId, size_t>>& rename);

}  // namespace op
}  // namespace ug
