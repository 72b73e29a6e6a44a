// op::Kernel -> ssa::Kernel.  Mirrors ug-core/src/lower_op.rs: the exact instruction shapes
// (index arithmetic, reduce idiom, loop order) are what a backend receives through
// Device::compile, so they are reproduced rule for rule.
#include <map>
#include <memory>

#include "block.h"
#include "lang.h"

namespace ug {
namespace op {

using block::Block;
using block::Id;

namespace {

// lower_op.rs:50-117
struct IndexFormula {
  enum Kind { kId, kConst, kAdd, kMul, kDiv, kMod } kind = kConst;
  Id id;
  size_t c = 0;  // Const value, or the rhs of Mul/Div/Mod
  std::shared_ptr<IndexFormula> lhs, rhs;

  static IndexFormula from_id(Id id) {
    IndexFormula f;
    f.kind = kId;
    f.id = id;
    return f;
  }
  static IndexFormula from_const(size_t c) {
    IndexFormula f;
    f.kind = kConst;
    f.c = c;
    return f;
  }
  IndexFormula add(const IndexFormula& r) const {
    IndexFormula f;
    f.kind = kAdd;
    f.lhs = std::make_shared<IndexFormula>(*this);
    f.rhs = std::make_shared<IndexFormula>(r);
    return f;
  }
  IndexFormula with(Kind k, size_t v) const {
    IndexFormula f;
    f.kind = k;
    f.c = v;
    f.lhs = std::make_shared<IndexFormula>(*this);
    return f;
  }
  IndexFormula mul(size_t v) const { return with(kMul, v); }
  IndexFormula div(size_t v) const { return with(kDiv, v); }
  IndexFormula mod(size_t v) const { return with(kMod, v); }

  // lower_op.rs:92-116: i32 index arithmetic.
  Id eval(Block& b) const {
    switch (kind) {
      case kId: return id;
      case kConst: return b.cst(Const::i32((int32_t)c));
      case kAdd: {
        Id l = lhs->eval(b);
        Id r = rhs->eval(b);
        return b.binary(BinaryOp::Add, l.to_a(), r.to_a(), DType::I32);
      }
      case kMul: {
        Id l = lhs->eval(b);
        return b.mul(l, (int32_t)c);
      }
      case kDiv: {
        if (c == 1) return lhs->eval(b);
        Id l = lhs->eval(b);
        return b.binary(BinaryOp::Div, l.to_a(), ssa::i32((int32_t)c), DType::I32);
      }
      case kMod: {
        if (c == 1) return b.cst(Const::i32(0));
        Id l = lhs->eval(b);
        return b.binary(BinaryOp::Mod, l.to_a(), ssa::i32((int32_t)c), DType::I32);
      }
    }
    bail("unreachable");
  }
};

using Indexes = std::vector<IndexFormula>;

template <typename T>
T take(std::vector<T>& v, size_t i) {
  T x = v[i];
  v.erase(v.begin() + (long)i);
  return x;
}

// lower_op.rs:127-202
Indexes layout_op(const Indexes& self, const LayoutOp& op, const Shape& shape, const Shape& arg_shape) {
  Indexes idxs = self;
  switch (op.kind) {
    case LayoutOp::Broadcast:
      for (size_t dim : op.broadcasted_dims) {
        if (dim >= idxs.size()) bail("unexpected dim for broadcast, " + std::to_string(dim) + " " + shape.str());
        idxs[dim] = IndexFormula::from_const(0);
      }
      for (size_t i = 0; i < op.inserted_dims; ++i) idxs.erase(idxs.begin());
      break;
    case LayoutOp::Narrow:
      if (op.dim >= idxs.size()) bail("unexpected dim for narrow, " + std::to_string(op.dim) + " " + shape.str());
      idxs[op.dim] = idxs[op.dim].add(IndexFormula::from_const(op.offset));
      break;
    case LayoutOp::Transpose:
      if (op.dim1 >= idxs.size() || op.dim2 >= idxs.size()) bail("unexpected dims for transpose " + shape.str());
      std::swap(idxs[op.dim1], idxs[op.dim2]);
      break;
    case LayoutOp::SplitDim: {
      if (op.dim >= arg_shape.rank()) bail("unexpected split dim " + std::to_string(op.dim) + " src " + shape.str());
      if (op.lhs >= shape.rank() || op.rhs >= shape.rank() || op.lhs == op.rhs) bail("unexpected split dims, dst " + shape.str());
      const auto& dims = shape.dims();
      IndexFormula l, r;
      if (op.lhs < op.rhs) {
        r = take(idxs, op.rhs);
        l = take(idxs, op.lhs);
      } else {
        l = take(idxs, op.lhs);
        r = take(idxs, op.rhs);
      }
      idxs.insert(idxs.begin() + (long)op.dim, l.mul(dims[op.rhs]).add(r));
      break;
    }
    case LayoutOp::MergeDims: {
      if (op.dim >= shape.rank()) bail("unexpected merge dim " + std::to_string(op.dim) + " dst " + shape.str());
      if (op.lhs >= arg_shape.rank() || op.rhs >= arg_shape.rank() || op.lhs == op.rhs) bail("unexpected merge dims, src " + arg_shape.str());
      const auto& ad = arg_shape.dims();
      IndexFormula idx = take(idxs, op.dim);
      // C layout: lhs is the slow dim, its stride is the size of rhs.
      IndexFormula lhs_idx = ad[op.lhs] <= 1 ? IndexFormula::from_const(0) : idx.div(ad[op.rhs]);
      IndexFormula rhs_idx = ad[op.rhs] <= 1 ? IndexFormula::from_const(0) : idx.mod(ad[op.rhs]);
      if (op.lhs < op.rhs) {
        idxs.insert(idxs.begin() + (long)op.lhs, lhs_idx);
        idxs.insert(idxs.begin() + (long)op.rhs, rhs_idx);
      } else {
        idxs.insert(idxs.begin() + (long)op.rhs, rhs_idx);
        idxs.insert(idxs.begin() + (long)op.lhs, lhs_idx);
      }
      break;
    }
  }
  return idxs;
}

// lower_op.rs:205-232: offset + sum idx * stride; `* 1` is elided, the running sum is the rhs.
std::pair<Id, Block> lower_layout(const ug::Layout& l, const Indexes& idxs) {
  if (idxs.size() != l.strides().size()) bail("len mismatch between strides and idxs");
  Block b;
  bool has_acc = false;
  Id acc{};
  if (l.offset() != 0) {
    acc = b.cst(Const::i32((int32_t)l.offset()));
    has_acc = true;
  }
  for (size_t k = 0; k < idxs.size(); ++k) {
    Id dim_id = idxs[k].eval(b);
    dim_id = b.mul(dim_id, (int32_t)l.strides()[k]);
    Id nid = has_acc ? b.binary(BinaryOp::Add, dim_id.to_a(), acc.to_a(), DType::I32) : dim_id;
    acc = nid;
    has_acc = true;
  }
  if (!has_acc) {
    Id id = Id::fresh();
    Block z;
    z.instrs.push_back({id, ssa::constant(Const::i32(0))});
    return {id, z};
  }
  return {acc, b};
}

// lower_op.rs:234-250
Const init_value(ReduceOp op, DType dt) {
  switch (op) {
    case ReduceOp::Sum: return Const::zero(dt);
    case ReduceOp::Min: return Const::max_value(dt);
    case ReduceOp::Max: return Const::min_value(dt);
  }
  bail("unreachable");
}
BinaryOp fold_op(ReduceOp op) { return op == ReduceOp::Sum ? BinaryOp::Add : (op == ReduceOp::Max ? BinaryOp::Max : BinaryOp::Min); }

// lower_op.rs:254-298: reductions over the same dim nested in the argument do not depend on the
// loop about to be opened; pull them out so they are evaluated once, before it.
Ast extract_const_walk(const Ast& ast, size_t tgt_dim, std::vector<std::pair<Id, Ast>>& accs) {
  const AstInner& in = *ast.inner;
  switch (in.kind) {
    case AstInner::Id:
    case AstInner::Load:
    case AstInner::Const: return ast;
    case AstInner::Reduce: {
      if (in.reduce_dim == tgt_dim) {
        Id src = Id::fresh();
        accs.push_back({src, ast});
        AstInner idn;
        idn.kind = AstInner::Id;
        idn.id_src = src.v;
        return make(std::move(idn), ast.dtype, ast.shape);
      }
      return reduce(in.reduce_op, extract_const_walk(in.arg, tgt_dim, accs), in.reduce_dim);
    }
    case AstInner::Unary: return unary(in.unary_op, extract_const_walk(in.arg, tgt_dim, accs), in.cast_to);
    case AstInner::Binary: {
      Ast l = extract_const_walk(in.arg, tgt_dim, accs);
      Ast r = extract_const_walk(in.rhs, tgt_dim, accs);
      return binary(in.binary_op, l, r);
    }
    case AstInner::Layout: {
      AstInner n;
      n.kind = AstInner::Layout;
      n.layout_op = in.layout_op;
      n.arg = extract_const_walk(in.arg, tgt_dim, accs);
      return make(std::move(n), ast.dtype, ast.shape);
    }
  }
  bail("unreachable");
}

using PerArg = std::map<size_t, uint32_t>;

// lower_op.rs:300-406
std::pair<Id, Block> lower_ast(const Ast& ast, const Indexes& idxs, const Opts& opts, const PerArg& per_arg) {
  const AstInner& in = *ast.inner;
  DType dtype = ast.dtype;
  switch (in.kind) {
    case AstInner::Load: {
      Id dst = Id::fresh();
      auto it = per_arg.find(in.load_src.v);
      if (it == per_arg.end()) bail("unknown arg " + std::to_string(in.load_src.v));
      auto off = lower_layout(in.load_layout, idxs);
      off.second.instrs.push_back({dst, ssa::load(it->second, off.first.to_a(), dtype)});
      return {dst, off.second};
    }
    case AstInner::Layout: {
      Indexes sub = layout_op(idxs, in.layout_op, ast.shape, in.arg.shape);
      return lower_ast(in.arg, sub, opts, per_arg);
    }
    case AstInner::Const: {
      Id dst = Id::fresh();
      Block b;
      b.instrs.push_back({dst, ssa::constant(in.cst)});
      return {dst, b};
    }
    case AstInner::Unary: {
      Id dst = Id::fresh();
      auto a = lower_ast(in.arg, idxs, opts, per_arg);
      a.second.instrs.push_back({dst, ssa::unary(in.unary_op, a.first.to_a(), dtype)});
      return {dst, a.second};
    }
    case AstInner::Reduce: {
      Id dst = Id::fresh();
      Block b;
      std::vector<std::pair<Id, Ast>> const_bits;
      Ast arg = extract_const_walk(in.arg, in.reduce_dim, const_bits);
      for (auto& cb : const_bits) {
        auto low = lower_ast(cb.second, idxs, opts, per_arg);
        b.extend(low.second);
        b.instrs.push_back({cb.first, ssa::unary(UnaryOp::Id, low.first.to_a(), cb.second.dtype)});
      }
      if (opts.has_thread_block && opts.thread_block.dim == in.reduce_dim && !(opts.has_block_axis && opts.block_axis == in.reduce_dim)) {
        auto low = lower_ast(arg, idxs, opts, per_arg);
        b.extend(low.second);
        b.instrs.push_back({dst, ssa::reduce_local(in.reduce_op, low.first.to_a(), dtype)});
      } else {
        b.instrs.push_back({dst, ssa::define_acc(init_value(in.reduce_op, dtype))});
        if (in.reduce_dim >= arg.shape.rank()) bail("unexpected dim for reduce, " + std::to_string(in.reduce_dim) + " " + ast.shape.str());
        size_t reduce_len = arg.shape.dims()[in.reduce_dim];
        block::Range r = b.range(ssa::i32(0), ssa::i32((int32_t)reduce_len), 1);
        Indexes ridx = idxs;
        if (in.reduce_dim >= ridx.size()) bail("reduce dim out of range of the index list");
        ridx[in.reduce_dim] = IndexFormula::from_id(r.id());
        auto low = lower_ast(arg, ridx, opts, per_arg);
        b.extend(low.second);
        Id src = b.push(ssa::binary(fold_op(in.reduce_op), dst.to_a(), low.first.to_a(), dtype));
        b.push(ssa::assign(dst.to_varid(), src.to_a()));
        b.end_range(r);
      }
      return {dst, b};
    }
    case AstInner::Binary: {
      Id dst = Id::fresh();
      auto l = lower_ast(in.arg, idxs, opts, per_arg);
      auto r = lower_ast(in.rhs, idxs, opts, per_arg);
      Block b;
      b.extend(l.second);
      b.extend(r.second);
      b.instrs.push_back({dst, ssa::binary(in.binary_op, l.first.to_a(), r.first.to_a(), dtype)});
      return {dst, b};
    }
    case AstInner::Id: return {Id{in.id_src}, Block()};
  }
  bail("unreachable");
}

}  // namespace

// lower_op.rs:409-491 + 537-557
ssa::Kernel Kernel::lower(const Opts& opts) const {
  Block b;
  PerArg per_arg;
  for (size_t index = 0; index < args.size(); ++index) {
    if (!args[index].is_ptr) bail("non-pointer arguments are not supported yet");
    Id id = b.push(ssa::define_global(index, args[index].dtype));
    per_arg[args[index].id.v] = id.to_varid();
  }
  Id block_id{}, thread_id{};
  if (opts.has_block_axis) block_id = b.push(ssa::special(UGHIP_SPECIAL_BLOCK_IDX));
  if (opts.has_thread_block) thread_id = b.push(ssa::special(UGHIP_SPECIAL_THREAD_IDX));

  for (const Store& st : ops) {
    auto pit = per_arg.find(st.dst.v);
    if (pit == per_arg.end()) bail("unknown arg " + std::to_string(st.dst.v));
    std::vector<block::Range> ranges;
    Indexes idxs;
    const auto& dims = st.layout.dims();
    for (size_t dim_idx = 0; dim_idx < dims.size(); ++dim_idx) {
      size_t len = dims[dim_idx];
      bool g = opts.has_block_axis && opts.block_axis == dim_idx;
      bool l = opts.has_thread_block && opts.thread_block.dim == dim_idx;
      Id id;
      if (g && l) {
        // Acts like an `if` rather than a `for`.
        Id gid = b.mul(block_id, (int32_t)opts.thread_block.block_dim);
        gid = b.binary(BinaryOp::Add, gid.to_a(), thread_id.to_a(), DType::I32);
        block::Range r = b.range(gid.to_a(), ssa::i32((int32_t)len), len);
        id = r.id();
        ranges.push_back(r);
      } else if (g) {
        id = block_id;
      } else if (l) {
        if (len == opts.thread_block.block_dim) {
          id = thread_id;
        } else {
          block::Range r = b.range(thread_id.to_a(), ssa::i32((int32_t)len), opts.thread_block.block_dim);
          id = r.id();
          ranges.push_back(r);
        }
      } else {
        block::Range r = b.range(ssa::i32(0), ssa::i32((int32_t)len), 1);
        id = r.id();
        ranges.push_back(r);
      }
      idxs.push_back(IndexFormula::from_id(id));
    }
    auto off = lower_layout(st.layout, idxs);
    b.extend(off.second);
    auto val = lower_ast(st.value, idxs, opts, per_arg);
    b.extend(val.second);
    b.push(ssa::store(pit->second, off.first.to_a(), val.first.to_a(), st.value.dtype));
    for (size_t k = ranges.size(); k-- > 0;) b.end_range(ranges[k]);
  }

  std::vector<ssa::Instr> instrs = b.relocate();
  std::vector<ughip_kernel_arg> kargs;
  for (size_t i = 0; i < args.size(); ++i) {
    ughip_kernel_arg a{};
    a.arg_id = args[i].id.v;
    a.is_ptr = 1;
    a.dtype = (uint8_t)args[i].dtype;
    a.var = (uint32_t)i;
    kargs.push_back(a);
  }
  uint32_t grid_dim = 1;
  if (opts.has_block_axis) {
    uint32_t local = opts.has_thread_block && opts.thread_block.dim == opts.block_axis ? (uint32_t)opts.thread_block.block_dim : 1;
    uint32_t len = !ops.empty() && opts.block_axis < ops[0].layout.rank() ? (uint32_t)ops[0].layout.dims()[opts.block_axis] : 1;
    grid_dim = (len + local - 1) / local;
  }
  uint32_t block_dim = opts.has_thread_block ? (uint32_t)opts.thread_block.block_dim : 1;
  return ssa::Kernel(std::move(instrs), std::move(kargs), LaunchConfig{grid_dim, block_dim, 0});
}

// lower_op.rs:636-664
namespace {
bool merge_walk(const Ast& ast) {
  const AstInner& in = *ast.inner;
  switch (in.kind) {
    case AstInner::Unary: return merge_walk(in.arg);
    case AstInner::Binary: return merge_walk(in.arg) && merge_walk(in.rhs);
    case AstInner::Load: return in.load_layout.can_be_compressed();
    case AstInner::Reduce: return false;
    case AstInner::Layout: return in.layout_op.kind == LayoutOp::Broadcast && in.layout_op.broadcasted_dims.size() >= ast.shape.rank();
    case AstInner::Const:
    case AstInner::Id: return true;
  }
  return false;
}

// lower_op.rs:494-526
Ast optimize_walk(const Ast& v) {
  const AstInner& in = *v.inner;
  switch (in.kind) {
    case AstInner::Unary: return unary(in.unary_op, optimize_walk(in.arg), in.cast_to);
    case AstInner::Binary: {
      Ast l = optimize_walk(in.arg);
      Ast r = optimize_walk(in.rhs);
      return binary(in.binary_op, l, r);
    }
    case AstInner::Load: return load(in.load_src, in.load_layout.compress_all(), v.dtype);
    case AstInner::Reduce: bail("unexpected result in optimize step");
    case AstInner::Layout:
      if (in.layout_op.kind != LayoutOp::Broadcast) bail("unexpected layout op in optimize step");
      return broadcast(optimize_walk(in.arg), Shape({v.shape.num_elements()}));
    case AstInner::Const:
    case AstInner::Id: return v;
  }
  bail("unreachable");
}
}  // namespace

bool Store::can_merge_all() const {
  if (!layout.can_be_compressed()) return false;
  return merge_walk(value);
}

Kernel Kernel::optimize() const {
  Kernel k = *this;
  for (Store& st : k.ops)
    if (st.can_merge_all()) {
      st.layout = st.layout.compress_all();
      st.value = optimize_walk(st.value);
    }
  return k;
}

// lower_op.rs:561-633: at most 40 characters describing the expression tree.
std::string Store::name() const {
  std::string chars;
  struct W {
    static void walk(const Ast& ast, std::string& c) {
      const AstInner& in = *ast.inner;
      switch (in.kind) {
        case AstInner::Unary: {
          char ch = 'i';
          switch (in.unary_op) {
            case UnaryOp::Id: ch = 'i'; break;
            case UnaryOp::Exp: ch = 'e'; break;
            case UnaryOp::Cos: ch = 'c'; break;
            case UnaryOp::Sin: ch = 's'; break;
            case UnaryOp::Neg: ch = 'n'; break;
            case UnaryOp::Sqrt: ch = 's'; break;
            case UnaryOp::Cast: ch = 'a'; break;
          }
          c += 'U';
          c += ch;
          c += '_';
          walk(in.arg, c);
          break;
        }
        case AstInner::Binary: {
          char ch = 'a';
          switch (in.binary_op) {
            case BinaryOp::Min: ch = 'n'; break;
            case BinaryOp::Max: ch = 'x'; break;
            case BinaryOp::Add: ch = 'a'; break;
            case BinaryOp::Sub: ch = 's'; break;
            case BinaryOp::Mul: ch = 'm'; break;
            case BinaryOp::Div: ch = 'd'; break;
            case BinaryOp::Mod: ch = 'o'; break;
          }
          c += 'B';
          c += ch;
          c += '_';
          walk(in.arg, c);
          c += '_';
          walk(in.rhs, c);
          break;
        }
        case AstInner::Load: c += 'O'; break;
        case AstInner::Reduce: {
          char ch = in.reduce_op == ReduceOp::Sum ? 's' : (in.reduce_op == ReduceOp::Max ? 'x' : 'n');
          c += 'R';
          c += ch;
          c += '_';
          walk(in.arg, c);
          break;
        }
        case AstInner::Layout: {
          char ch = 'b';
          switch (in.layout_op.kind) {
            case LayoutOp::Narrow: ch = 'n'; break;
            case LayoutOp::SplitDim: ch = 's'; break;
            case LayoutOp::MergeDims: ch = 'm'; break;
            case LayoutOp::Transpose: ch = 't'; break;
            case LayoutOp::Broadcast: ch = 'b'; break;
          }
          c += 'L';
          c += ch;
          c += '_';
          walk(in.arg, c);
          break;
        }
        case AstInner::Const: c += 'C'; break;
        case AstInner::Id: c += 'I'; break;
      }
    }
  };
  W::walk(value, chars);
  if (chars.size() > 40) chars.resize(40);
  return chars;
}

std::string ast_key(const Ast& ast, const std::vector<std::pair<ArgId, size_t>>& rename) {
  const AstInner& in = *ast.inner;
  std::string s = "(" + std::to_string((int)in.kind) + ";" + std::to_string((int)ast.dtype) + ";" + ast.shape.str() + ";";
  switch (in.kind) {
    case AstInner::Id: bail("unexpected id node");
    case AstInner::Load: {
      size_t idx = (size_t)-1;
      for (auto& p : rename)
        if (p.first == in.load_src) idx = p.second;
      if (idx == (size_t)-1) bail("BUG: missing arg id " + std::to_string(in.load_src.v));
      s += "a" + std::to_string(idx) + in.load_layout.key();
      break;
    }
    case AstInner::Reduce: s += "r" + std::to_string((int)in.reduce_op) + ":" + std::to_string(in.reduce_dim) + ast_key(in.arg, rename); break;
    case AstInner::Unary: s += "u" + std::to_string((int)in.unary_op) + ":" + std::to_string((int)in.cast_to) + ast_key(in.arg, rename); break;
    case AstInner::Binary: s += "b" + std::to_string((int)in.binary_op) + ast_key(in.arg, rename) + ast_key(in.rhs, rename); break;
    case AstInner::Const: s += in.cst.key(); break;
    case AstInner::Layout: s += in.layout_op.key() + ast_key(in.arg, rename); break;
  }
  return s + ")";
}

}  // namespace op
}  // namespace ug
