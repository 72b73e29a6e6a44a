// Scheduler: LazyBuffer DAG -> ordered kernels / matmuls / custom calls.  Mirrors
// ug-core/src/schedule.rs (fusion boundaries, argument order) and cache.rs.
#include <algorithm>
#include <set>
#include <unordered_map>

#include "lazy_buffer.h"

namespace ug {

// schedule.rs:23-39
op::Kernel KernelItem::kernel() const {
  op::Kernel k;
  k.name = "realize_" + std::to_string(dst.second.id());
  for (const auto& a : args) k.args.push_back(Arg{a.first, a.second.dtype(), true});
  op::Store st;
  st.dst = dst.first;
  st.layout = has_dst_layout ? dst_layout : Layout::from_shape(dst.second.shape());
  st.value = ast;
  k.ops.push_back(st);
  return k;
}

std::string normalized_kernel_key(const op::Kernel& k) {
  std::vector<std::pair<ArgId, size_t>> rename;
  std::string s;
  for (size_t i = 0; i < k.args.size(); ++i) {
    rename.push_back({k.args[i].id, i});
    s += "A" + std::to_string((int)k.args[i].dtype);
  }
  for (const op::Store& st : k.ops) {
    size_t idx = (size_t)-1;
    for (auto& p : rename)
      if (p.first == st.dst) idx = p.second;
    if (idx == (size_t)-1) bail("BUG: missing arg id");
    s += "|S" + std::to_string(idx) + st.layout.key() + op::ast_key(st.value, rename);
  }
  return s;
}

namespace {

// schedule.rs:480-520: use counts (1, or 2 for "twice or more"); realized nodes stop the walk.
void id_cnts(const LazyBuffer& b, std::unordered_map<size_t, size_t>& cnts) {
  if (b.realized()) return;
  size_t& cnt = cnts[b.id()];
  cnt += 1;
  if (cnt > 1) return;
  const Op& op = b.inner().op;
  switch (op.kind) {
    case Op::Value:
    case Op::Const: break;
    case Op::Reshape:
    case Op::Layout:
    case Op::Reduce:
    case Op::Unary: id_cnts(op.arg, cnts); break;
    case Op::Set:
      id_cnts(op.arg2, cnts);  // src
      id_cnts(op.arg, cnts);   // values
      break;
    case Op::MatMul:
    case Op::Binary:
      id_cnts(op.arg, cnts);
      id_cnts(op.arg2, cnts);
      break;
    case Op::CustomIp:
      for (const LazyBuffer& a : op.args) id_cnts(a, cnts);
      id_cnts(op.arg2, cnts);
      break;
    case Op::Ssa:
    case Op::Custom:
      for (const LazyBuffer& a : op.args) id_cnts(a, cnts);
      break;
  }
}

// schedule.rs:308-475
struct Context {
  std::vector<ScheduleItem> items;
  std::map<size_t, LazyBuffer> per_arg_id;
  std::unordered_map<size_t, op::Ast> ast_cache;
  std::unordered_map<size_t, size_t> cnts;

  const LazyBuffer& get_arg_id(ArgId id) const {
    auto it = per_arg_id.find(id.v);
    if (it == per_arg_id.end()) bail("no arg for id " + std::to_string(id.v));
    return it->second;
  }

  ArgId new_arg(const LazyBuffer& b) {
    ArgId id = ArgId::fresh();
    per_arg_id[id.v] = b;
    return id;
  }

  op::Ast walk(const LazyBuffer& b) {
    size_t id = b.id();
    auto cached = ast_cache.find(id);
    if (cached != ast_cache.end()) return cached->second;
    DType dtype = b.dtype();
    const Shape& shape = b.shape();
    op::Ast ast;
    if (b.realized()) {
      ast = op::load(new_arg(b), Layout::from_shape(shape), dtype);
    } else {
      const Op& op = b.inner().op;
      switch (op.kind) {
        case Op::Unary: ast = op::unary(op.unary_op, walk(op.arg), op.cast_to); break;
        case Op::Binary: {
          op::Ast l = walk(op.arg);
          op::Ast r = walk(op.arg2);
          ast = op::binary(op.binary_op, l, r);
          break;
        }
        case Op::MatMul: {
          // Matmuls are not fused: both operands are materialised by their own kernels.
          push_schedule_item(op.arg);
          push_schedule_item(op.arg2);
          ArgId dst_id = new_arg(b);
          ScheduleItem it;
          it.kind = ScheduleItem::MatMul;
          it.dst = b;
          it.lhs = op.arg;
          it.rhs = op.arg2;
          it.b = op.b;
          it.m = op.m;
          it.n = op.n;
          it.k = op.k;
          it.transpose = op.transpose;
          items.push_back(std::move(it));
          ast = op::load(dst_id, Layout::from_shape(shape), dtype);
          break;
        }
        case Op::Reduce: ast = op::reduce(op.reduce_op, walk(op.arg), op.reduce_dim); break;
        case Op::Const: ast = op::cst(op.cst); break;
        case Op::Value: ast = op::load(new_arg(b), Layout::from_shape(shape), dtype); break;
        case Op::Reshape: {
          ArgId dst_id = push_schedule_item(op.arg);
          ast = op::load(dst_id, Layout::from_shape(shape), dtype);
          break;
        }
        case Op::Layout: ast = op::layout(op.layout_op, walk(op.arg), shape); break;
        case Op::Ssa: {
          Args args;
          for (const LazyBuffer& a : op.args) args.push_back({push_schedule_item(a), a});
          ArgId dst_id = new_arg(b);
          args.push_back({dst_id, b});
          ScheduleItem it;
          it.kind = ScheduleItem::Ssa;
          it.ssa = op.ssa;
          it.args = std::move(args);
          items.push_back(std::move(it));
          ast = op::load(dst_id, Layout::from_shape(shape), dtype);
          break;
        }
        case Op::Set: {
          ArgId arg_id = push_schedule_item(op.arg2);
          op::Ast values = walk(op.arg);
          push_kernel(op.arg2, values, &op.dst_layout);
          ast = op::load(arg_id, Layout::from_shape(shape), dtype);
          break;
        }
        case Op::CustomIp: {
          Args args;
          for (const LazyBuffer& a : op.args) args.push_back({push_schedule_item(a), a});
          ArgId arg_id = push_schedule_item(op.arg2);
          args.push_back({arg_id, op.arg2});
          ScheduleItem it;
          it.kind = ScheduleItem::Custom;
          it.f = op.f;
          it.args = std::move(args);
          items.push_back(std::move(it));
          ast = op::load(arg_id, Layout::from_shape(shape), dtype);
          break;
        }
        case Op::Custom: {
          Args args;
          for (const LazyBuffer& a : op.args) args.push_back({push_schedule_item(a), a});
          ArgId dst_id = new_arg(b);
          args.push_back({dst_id, b});
          ScheduleItem it;
          it.kind = ScheduleItem::Custom;
          it.f = op.f;
          it.args = std::move(args);
          items.push_back(std::move(it));
          ast = op::load(dst_id, Layout::from_shape(shape), dtype);
          break;
        }
      }
    }
    // A subtree used more than once gets a kernel of its own (schedule.rs:429-435).
    auto c = cnts.find(id);
    if (c != cnts.end() && c->second > 1) {
      ArgId dst_id = push_kernel(b, ast, nullptr);
      ast = op::load(dst_id, Layout::from_shape(shape), dtype);
    }
    ast_cache[id] = ast;
    return ast;
  }

  ArgId push_kernel(const LazyBuffer& buffer, const op::Ast& ast, const Layout* dst_layout) {
    if (ast.inner->kind == op::AstInner::Load) {
      const LazyBuffer& src = get_arg_id(ast.inner->load_src);
      // Loading and immediately storing the same buffer is a no-op (schedule.rs:446-453).
      if (src.data().get() == buffer.data().get()) return ast.inner->load_src;
    }
    ArgId dst_id = new_arg(buffer);
    std::set<ArgId> ids;
    op::arg_ids(ast, ids);
    ids.insert(dst_id);
    ScheduleItem it;
    it.kind = ScheduleItem::Kernel;
    for (const ArgId& a : ids) it.kernel.args.push_back({a, get_arg_id(a)});
    it.kernel.ast = ast;
    it.kernel.dst = {dst_id, buffer};
    if (dst_layout) {
      it.kernel.has_dst_layout = true;
      it.kernel.dst_layout = *dst_layout;
    }
    items.push_back(std::move(it));
    return dst_id;
  }

  ArgId push_schedule_item(const LazyBuffer& buffer) {
    op::Ast ast = walk(buffer);
    return push_kernel(buffer, ast, nullptr);
  }
};

}  // namespace

Schedule Schedule::create(const std::vector<LazyBuffer>& buffers) {
  if (buffers.empty()) bail("no buffers provided");
  Context ctx;
  for (const LazyBuffer& b : buffers) id_cnts(b, ctx.cnts);
  for (const LazyBuffer& b : buffers) ctx.push_schedule_item(b);
  Schedule s;
  s.device_ = buffers[0].device();
  s.items_ = std::move(ctx.items);
  s.per_arg_id_ = std::move(ctx.per_arg_id);
  return s;
}

const LazyBuffer& Schedule::get_arg_id(ArgId id) const {
  auto it = per_arg_id_.find(id.v);
  if (it == per_arg_id_.end()) bail("no arg for id " + std::to_string(id.v));
  return it->second;
}

// schedule.rs:115-207
CompiledSchedule Schedule::compile_with_cache(CompilationCache& cache) const {
  CompiledSchedule out;
  out.device = device_;
  for (const ScheduleItem& item : items_) out.funcs.push_back(compile_item(item, cache));
  return out;
}

CompiledSchedule Schedule::compile_and_run(CompilationCache& cache) const {
  CompiledSchedule out;
  out.device = device_;
  out.funcs.reserve(items_.size());
  for (const ScheduleItem& item : items_) {
    out.funcs.push_back(compile_item(item, cache));
    out.run_one(out.funcs.back());
  }
  return out;
}

CompiledFunc Schedule::compile_item(const ScheduleItem& item, CompilationCache& cache) const {
  {
    CompiledFunc call;
    switch (item.kind) {
      case ScheduleItem::MatMul:
        call.kind = CompiledFunc::MatMul;
        call.dst = item.dst;
        call.lhs = item.lhs;
        call.rhs = item.rhs;
        call.b = item.b;
        call.m = item.m;
        call.n = item.n;
        call.k = item.k;
        call.transpose = item.transpose;
        break;
      case ScheduleItem::Custom:
        call.kind = CompiledFunc::Custom;
        call.f = item.f;
        call.args = item.args;
        break;
      case ScheduleItem::Ssa: {
        call.kind = CompiledFunc::Kernel;
        call.args = item.args;
        std::string key = item.ssa.instrs_key();
        auto it = cache.ssa_cache.find(key);
        if (it != cache.ssa_cache.end()) {
          call.func = it->second;
        } else {
          call.func = device_->compile(item.ssa, nullptr);
          cache.ssa_cache[key] = call.func;
        }
        break;
      }
      case ScheduleItem::Kernel: {
        call.kind = CompiledFunc::Kernel;
        op::Kernel kernel = item.kernel.kernel();
        std::string key = normalized_kernel_key(kernel);
        for (const Arg& a : kernel.args) call.args.push_back({a.id, get_arg_id(a.id)});
        auto it = cache.op_cache.find(key);
        if (it != cache.op_cache.end()) {
          call.func = it->second;
          break;
        }
        std::string kernel_name = kernel.ops.empty() ? "" : kernel.ops[0].name();
        kernel = kernel.optimize();
        op::Opts opts;
        // schedule.rs:162-188: grid heuristics, only for devices that ask for them.
        if (device_->use_grid() && kernel.ops.size() == 1 && kernel.ops[0].layout.rank() >= 1 && kernel.ops[0].layout.num_elements() >= 1) {
          std::vector<std::pair<size_t, size_t>> dims;
          for (size_t i = 0; i < kernel.ops[0].layout.rank(); ++i) dims.push_back({i, kernel.ops[0].layout.dims()[i]});
          std::stable_sort(dims.begin(), dims.end(), [](const auto& a, const auto& b) { return a.second > b.second; });
          if (dims.size() >= 2 && dims[1].second > 1) opts = op::Opts().with_block_axis(dims[0].first).with_thread_block(dims[1].first, 32);
          else if (dims.size() > 1 && dims[0].second > 1) opts = op::Opts().with_global_axis(dims[0].first, 32);
        }
        ssa::Kernel ssa = kernel.lower(opts);
        call.func = device_->compile(ssa, kernel.ops.empty() ? nullptr : &kernel_name);
        cache.op_cache[key] = call.func;
        break;
      }
    }
    return call;
  }
}

void CompiledSchedule::allocate_all() const {
  for (const CompiledFunc& f : funcs) {
    if (f.kind == CompiledFunc::MatMul) {
      f.dst.maybe_allocate_uninit();
      f.lhs.maybe_allocate_uninit();
      f.rhs.maybe_allocate_uninit();
    } else {
      for (const auto& a : f.args) a.second.maybe_allocate_uninit();
    }
  }
}

// schedule.rs:234-305
void CompiledSchedule::run() const {
  for (const CompiledFunc& f : funcs) run_one(f);
}

void CompiledSchedule::run_one(const CompiledFunc& f) const {
  thread_local std::vector<Slice*> bs;
  {
    switch (f.kind) {
      case CompiledFunc::Kernel:
      case CompiledFunc::Custom: {
        bs.clear();
        for (const auto& a : f.args) {
          a.second.maybe_allocate_uninit();
          // RefCell::try_borrow_mut: a cell may appear once.
          Slice* s = a.second.data()->slice.get();
          for (Slice* seen : bs)
            if (seen == s) bail("already borrowed: BorrowMutError");
          bs.push_back(s);
        }
        if (f.kind == CompiledFunc::Kernel) device->run(*f.func, bs);
        else (*f.f)(bs);
        break;
      }
      case CompiledFunc::MatMul: {
        const auto& ld = f.lhs.dims();
        const auto& rd = f.rhs.dims();
        size_t lr = ld.size(), rr = rd.size();
        std::vector<size_t> lp(ld), rp(rd);
        if (lr < rr) lp.insert(lp.begin(), rr - lr, 1);
        if (rr < lr) rp.insert(rp.begin(), lr - rr, 1);
        Layout lhs_l = Layout::from_shape(Shape(lp));
        Layout rhs_l = Layout::from_shape(Shape(rp));
        if (f.transpose) rhs_l = rhs_l.transpose();
        f.dst.maybe_allocate_uninit();
        f.lhs.maybe_allocate_uninit();
        f.rhs.maybe_allocate_uninit();
        if (f.dst.data().get() == f.lhs.data().get() || f.dst.data().get() == f.rhs.data().get()) bail("already borrowed: BorrowMutError");
        device->matmul(*f.dst.data()->slice, *f.lhs.data()->slice, *f.rhs.data()->slice, f.b, f.m, f.n, f.k, lhs_l, rhs_l);
        break;
      }
    }
  }
}

}  // namespace ug
