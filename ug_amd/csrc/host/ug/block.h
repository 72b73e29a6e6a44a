// Block builder: ssa instructions with explicit destination ids, relocated to line numbers at
// the end.  Mirrors ug-core/src/block.rs.
#pragma once
#include <unordered_map>
#include <utility>
#include <vector>

#include "lang.h"

namespace ug {
namespace block {

// block.rs:7-29.  Ids only need to be unique inside one kernel.
struct Id {
  uint32_t v = 0;
  static Id fresh() {
    static std::atomic<uint32_t> counter{1};
    return Id{counter.fetch_add(1)};
  }
  ssa::A to_a() const { return ssa::var(v); }
  uint32_t to_varid() const { return v; }
};

struct Range {
  Id range_id, erange_id;
  Id id() const { return range_id; }
};

// block.rs:39-223
struct Block {
  std::vector<std::pair<Id, ssa::Instr>> instrs;

  Range range(ssa::A lo, ssa::A up, size_t step) {
    Range r{Id::fresh(), Id::fresh()};
    instrs.push_back({r.range_id, ssa::range(lo, up, step, r.erange_id.v)});
    return r;
  }
  void end_range(const Range& r) { instrs.push_back({r.erange_id, ssa::end_range(r.range_id.v)}); }

  Id push(const ssa::Instr& in) {
    Id id = Id::fresh();
    instrs.push_back({id, in});
    return id;
  }
  // block.rs:68-102: `+ 0` and `* 1` are elided.
  Id add(Id src, int32_t v) {
    if (v == 0) return src;
    return push(ssa::binary(BinaryOp::Add, src.to_a(), ssa::i32(v), DType::I32));
  }
  Id mul(Id src, int32_t v) {
    if (v == 1) return src;
    return push(ssa::binary(BinaryOp::Mul, src.to_a(), ssa::i32(v), DType::I32));
  }
  Id cst(const Const& c) { return push(ssa::constant(c)); }
  Id unary(UnaryOp op, ssa::A arg, DType dt) { return push(ssa::unary(op, arg, dt)); }
  Id binary(BinaryOp op, ssa::A lhs, ssa::A rhs, DType dt) { return push(ssa::binary(op, lhs, rhs, dt)); }
  void extend(const Block& o) { instrs.insert(instrs.end(), o.instrs.begin(), o.instrs.end()); }

  // block.rs:143-222: unique ids -> line numbers.
  std::vector<ssa::Instr> relocate() const {
    std::unordered_map<uint32_t, uint32_t> per_id;
    for (size_t line = 0; line < instrs.size(); ++line) per_id[instrs[line].first.v] = (uint32_t)line;
    auto get_id = [&](uint32_t id) {
      auto it = per_id.find(id);
      if (it == per_id.end()) bail("id not found " + std::to_string(id));
      return it->second;
    };
    auto get_a = [&](ssa::A a) {
      if (!a.is_const) a.var = get_id(a.var);
      return a;
    };
    std::vector<ssa::Instr> out;
    out.reserve(instrs.size());
    for (const auto& p : instrs) {
      ssa::Instr in = p.second;
      switch (in.op) {
        case UGHIP_I_STORE:
          in.v = get_id(in.v);
          in.a = get_a(in.a);
          in.b = get_a(in.b);
          break;
        case UGHIP_I_IF:
          in.a = get_a(in.a);
          in.v = get_id(in.v);
          break;
        case UGHIP_I_RANGE:
          in.a = get_a(in.a);
          in.b = get_a(in.b);
          in.v = get_id(in.v);
          break;
        case UGHIP_I_LOAD:
          in.v = get_id(in.v);
          in.a = get_a(in.a);
          break;
        case UGHIP_I_BINARY:
          in.a = get_a(in.a);
          in.b = get_a(in.b);
          break;
        case UGHIP_I_UNARY:
        case UGHIP_I_REDUCE_LOCAL: in.a = get_a(in.a); break;
        case UGHIP_I_ASSIGN:
          in.v = get_id(in.v);
          in.a = get_a(in.a);
          break;
        case UGHIP_I_END_RANGE: in.v = get_id(in.v); break;
        default: break;
      }
      out.push_back(in);
    }
    return out;
  }
};

}  // namespace block
}  // namespace ug
