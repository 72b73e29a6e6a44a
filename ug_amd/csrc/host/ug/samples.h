// Hand-written kernels used as fixtures.  Mirrors ug-core/src/samples.rs:1-256: the same
// instruction sequences, so the reference's golden vectors (ug-core/tests/basic_tests.rs)
// apply unchanged.
#pragma once
#include "block.h"
#include "lang.h"

namespace ug {
namespace samples {
namespace ssa_k {

using ssa::Instr;
using ssa::var;
inline ssa::A i32(int32_t v) { return ssa::i32(v); }
inline Instr arg(size_t index, DType dt) { return ssa::define_global(index, dt); }

// samples.rs:10-27
inline ssa::Kernel simple_add(size_t vec_len) {
  DType dt = DType::I32;
  std::vector<Instr> in = {
      arg(0, dt),
      arg(1, dt),
      arg(2, dt),
      ssa::range(i32(0), i32((int32_t)vec_len), 1, 8),
      ssa::load(1, var(3), dt),
      ssa::load(2, var(3), dt),
      ssa::binary(BinaryOp::Add, var(4), var(5), dt),
      ssa::store(0, var(3), var(6), dt),
      ssa::end_range(3),
  };
  return ssa::Kernel::from_instrs(in);
}

// samples.rs:29-50
inline ssa::Kernel simple_dotprod(size_t vec_len) {
  DType dt = DType::F32;
  std::vector<Instr> in = {
      arg(0, dt),
      arg(1, dt),
      arg(2, dt),
      ssa::constant(Const::i32(0)),
      ssa::constant(Const::i32((int32_t)vec_len)),
      ssa::define_acc(Const::f32(0.f)),
      ssa::range(var(3), var(4), 1, 12),
      ssa::load(1, var(6), dt),
      ssa::load(2, var(6), dt),
      ssa::binary(BinaryOp::Mul, var(7), var(8), dt),
      ssa::binary(BinaryOp::Add, var(9), var(5), dt),
      ssa::assign(5, var(10)),
      ssa::end_range(6),
      ssa::store(0, var(3), var(5), dt),
  };
  return ssa::Kernel::from_instrs(in);
}

// samples.rs:52-71
inline ssa::Kernel exp(size_t block_size) {
  block::Block b;
  DType dt = DType::F32;
  auto src = b.push(arg(0, dt));
  auto dst = b.push(arg(1, dt));
  auto g = b.push(ssa::special(UGHIP_SPECIAL_BLOCK_IDX));
  auto l = b.push(ssa::special(UGHIP_SPECIAL_THREAD_IDX));
  auto off = b.mul(g, (int32_t)block_size);
  off = b.binary(BinaryOp::Add, off.to_a(), l.to_a(), DType::I32);
  auto ld = b.push(ssa::load(src.v, off.to_a(), dt));
  auto val = b.unary(UnaryOp::Exp, ld.to_a(), dt);
  b.push(ssa::store(dst.v, off.to_a(), val.to_a(), dt));
  return ssa::Kernel::from_instrs(b.relocate());
}

// samples.rs:73-99
inline ssa::Kernel exp_block(size_t dim2, size_t block_size) {
  if (dim2 % block_size != 0) bail("last-dim must be divisible by block size");
  block::Block b;
  DType dt = DType::F32;
  auto src = b.push(arg(0, dt));
  auto dst = b.push(arg(1, dt));
  auto g = b.push(ssa::special(UGHIP_SPECIAL_BLOCK_IDX));
  auto l = b.push(ssa::special(UGHIP_SPECIAL_THREAD_IDX));
  auto base = b.mul(g, (int32_t)dim2);
  base = b.binary(BinaryOp::Add, base.to_a(), l.to_a(), DType::I32);
  for (size_t i = 0; i < dim2; i += block_size) {
    auto off = b.add(base, (int32_t)i);
    auto ld = b.push(ssa::load(src.v, off.to_a(), dt));
    auto val = b.unary(UnaryOp::Exp, ld.to_a(), dt);
    b.push(ssa::store(dst.v, off.to_a(), val.to_a(), dt));
  }
  return ssa::Kernel::from_instrs(b.relocate());
}

// samples.rs:101-158: LDS tree reduction with barriers; dim2 must be a power of two.
inline ssa::Kernel softmax_barrier(size_t, size_t dim2) {
  block::Block b;
  DType dt = DType::F32;
  auto src = b.push(arg(0, dt));
  auto dst = b.push(arg(1, dt));
  auto sto = b.push(ssa::define_local(2 * dim2, dt));
  auto g = b.push(ssa::special(UGHIP_SPECIAL_BLOCK_IDX));
  auto l = b.push(ssa::special(UGHIP_SPECIAL_THREAD_IDX));
  auto base = b.mul(g, (int32_t)dim2);
  auto goff = b.binary(BinaryOp::Add, base.to_a(), l.to_a(), DType::I32);
  auto ld = b.push(ssa::load(src.v, goff.to_a(), dt));

  b.push(ssa::store(sto.v, l.to_a(), ld.to_a(), dt));
  b.push(ssa::barrier());
  auto v = ld;
  for (size_t offset = 1; offset < dim2; offset *= 2) {
    auto off = b.add(l, (int32_t)offset);
    auto m = b.push(ssa::load(sto.v, off.to_a(), dt));
    v = b.binary(BinaryOp::Max, m.to_a(), v.to_a(), dt);
    b.push(ssa::store(sto.v, l.to_a(), v.to_a(), dt));
    b.push(ssa::barrier());
  }
  auto mx = b.push(ssa::load(sto.v, i32(0), dt));
  auto val = b.binary(BinaryOp::Sub, ld.to_a(), mx.to_a(), dt);
  val = b.unary(UnaryOp::Exp, val.to_a(), dt);

  b.push(ssa::store(sto.v, l.to_a(), val.to_a(), dt));
  b.push(ssa::barrier());
  v = val;
  for (size_t offset = 1; offset < dim2; offset *= 2) {
    auto off = b.add(l, (int32_t)offset);
    auto m = b.push(ssa::load(sto.v, off.to_a(), dt));
    v = b.binary(BinaryOp::Add, m.to_a(), v.to_a(), dt);
    b.push(ssa::store(sto.v, l.to_a(), v.to_a(), dt));
    b.push(ssa::barrier());
  }
  auto sum = b.push(ssa::load(sto.v, i32(0), dt));
  val = b.binary(BinaryOp::Div, val.to_a(), sum.to_a(), dt);
  b.push(ssa::store(dst.v, goff.to_a(), val.to_a(), dt));
  return ssa::Kernel::from_instrs(b.relocate());
}

// samples.rs:160-183
inline ssa::Kernel softmax_reduce(size_t, size_t dim2) {
  block::Block b;
  DType dt = DType::F32;
  auto src = b.push(arg(0, dt));
  auto dst = b.push(arg(1, dt));
  auto g = b.push(ssa::special(UGHIP_SPECIAL_BLOCK_IDX));
  auto l = b.push(ssa::special(UGHIP_SPECIAL_THREAD_IDX));
  auto base = b.mul(g, (int32_t)dim2);
  auto goff = b.binary(BinaryOp::Add, base.to_a(), l.to_a(), DType::I32);
  auto ld = b.push(ssa::load(src.v, goff.to_a(), dt));
  auto mx = b.push(ssa::reduce_local(ReduceOp::Max, ld.to_a(), dt));
  auto val = b.binary(BinaryOp::Sub, ld.to_a(), mx.to_a(), dt);
  val = b.unary(UnaryOp::Exp, val.to_a(), dt);
  auto sum = b.push(ssa::reduce_local(ReduceOp::Sum, val.to_a(), dt));
  val = b.binary(BinaryOp::Div, val.to_a(), sum.to_a(), dt);
  b.push(ssa::store(dst.v, goff.to_a(), val.to_a(), dt));
  return ssa::Kernel::from_instrs(b.relocate());
}

// samples.rs:185-228
inline ssa::Kernel softmax_block(size_t, size_t dim2, size_t block_size) {
  if (dim2 % block_size != 0) bail("last-dim must be divisible by block size");
  block::Block b;
  DType dt = DType::F32;
  auto src = b.push(arg(0, dt));
  auto dst = b.push(arg(1, dt));
  auto g = b.push(ssa::special(UGHIP_SPECIAL_BLOCK_IDX));
  auto l = b.push(ssa::special(UGHIP_SPECIAL_THREAD_IDX));
  auto base = b.mul(g, (int32_t)dim2);
  auto goff = b.binary(BinaryOp::Add, base.to_a(), l.to_a(), DType::I32);
  std::vector<block::Id> loads, values;
  auto mx = b.push(ssa::constant(Const::f32(-INFINITY)));
  for (size_t i = 0; i < dim2; i += block_size) {
    auto off = b.add(goff, (int32_t)i);
    auto ld = b.push(ssa::load(src.v, off.to_a(), dt));
    mx = b.binary(BinaryOp::Max, mx.to_a(), ld.to_a(), dt);
    loads.push_back(ld);
  }
  mx = b.push(ssa::reduce_local(ReduceOp::Max, mx.to_a(), dt));
  auto sum = b.push(ssa::constant(Const::i32(0)));
  for (auto ld : loads) {
    auto val = b.binary(BinaryOp::Sub, ld.to_a(), mx.to_a(), dt);
    val = b.unary(UnaryOp::Exp, val.to_a(), dt);
    sum = b.binary(BinaryOp::Add, val.to_a(), sum.to_a(), dt);
    values.push_back(val);
  }
  sum = b.push(ssa::reduce_local(ReduceOp::Sum, sum.to_a(), dt));
  for (size_t k = 0; k < values.size(); ++k) {
    auto off = b.add(goff, (int32_t)(k * block_size));
    auto val = b.binary(BinaryOp::Div, values[k].to_a(), sum.to_a(), dt);
    b.push(ssa::store(dst.v, off.to_a(), val.to_a(), dt));
  }
  return ssa::Kernel::from_instrs(b.relocate());
}

}  // namespace ssa_k

// samples.rs:239-255: softmax as one fused op-level kernel.
inline op::Kernel op_softmax(size_t dim1, size_t dim2) {
  Layout layout = Layout::from_shape(Shape({dim1, dim2}));
  Arg src_ptr = Arg::ptr(DType::F32), dst_ptr = Arg::ptr(DType::F32);
  op::Ast src = op::load(src_ptr.id, layout, DType::F32);
  op::Ast mx = op::broadcast(op::reduce(ReduceOp::Max, src, 1), Shape({dim1, dim2}));
  op::Ast e = op::unary(UnaryOp::Exp, op::binary(BinaryOp::Sub, src, mx));
  op::Ast se = op::broadcast(op::reduce(ReduceOp::Sum, e, 1), Shape({dim1, dim2}));
  op::Ast sm = op::binary(BinaryOp::Div, e, se);
  op::Kernel k;
  k.name = "softmax_" + std::to_string(dim1) + "_" + std::to_string(dim2);
  k.args = {src_ptr, dst_ptr};
  k.ops = {op::Store{dst_ptr.id, layout, sm}};
  return k;
}

// basic_tests.rs:118-136: (x - 0.5) * 3 in place.
inline op::Kernel op_affine(size_t n) {
  Layout layout = Layout::from_shape(Shape({n}));
  Arg ptr = Arg::ptr(DType::F32);
  op::Ast src = op::load(ptr.id, layout, DType::F32);
  op::Ast sub = op::broadcast_binary(BinaryOp::Sub, src, op::cst(Const::f32(0.5f)));
  op::Ast mul = op::broadcast_binary(BinaryOp::Mul, sub, op::cst(Const::f32(3.f)));
  op::Kernel k;
  k.name = "affine";
  k.args = {ptr};
  k.ops = {op::Store{ptr.id, layout, mul}};
  return k;
}

}  // namespace samples
}  // namespace ug
