// ORACLE -- TEST INFRASTRUCTURE ONLY.
// Lane-vector SSA interpreter: restatement of ug-core/src/interpreter.rs:201-435.  N lanes stand
// for the threads of one block and step in lock-step; divergent control flow is an error
// (:232-234, :261-263); ReduceLocal folds over all lanes (:392-413); arithmetic exists for f32
// and i32 only, anything else is a "dtype mismatch" like in the reference.  A GPU-free check of
// SSA semantics, pinned by ug-core/tests/basic_tests.rs.
#include <algorithm>
#include <cmath>

#include "oracle.h"

namespace ug_oracle {

using namespace ug;

namespace {

struct Value {
  enum Kind { None, Ptr, LocalPtr, F32, I32 } kind = None;
  size_t buf = 0;
  std::vector<float> f;
  std::vector<int32_t> i;
};

struct Local {
  DType dtype;
  std::vector<float> f;
  std::vector<int32_t> i;
};

}  // namespace

void eval_ssa(const ssa::Kernel& kernel, std::vector<InterpBuffer>& buffers, size_t N, size_t grid_idx) {
  const auto& instrs = kernel.instrs;
  std::vector<Value> values(instrs.size());
  std::vector<Local> locals;
  auto splat_f = [&](float x) {
    Value v;
    v.kind = Value::F32;
    v.f.assign(N, x);
    return v;
  };
  auto splat_i = [&](int32_t x) {
    Value v;
    v.kind = Value::I32;
    v.i.assign(N, x);
    return v;
  };
  auto from_const = [&](const ughip_a& a) -> Value {
    switch (a.dtype) {
      case UGHIP_F32: return splat_f(a.f);
      case UGHIP_I32: return splat_i((int32_t)a.i);
      default: bail("interpreter: unsupported const dtype");
    }
  };
  auto get = [&](const ughip_a& a) -> Value {
    if (a.is_const) return from_const(a);
    if (a.var >= values.size()) bail("get out of bound " + std::to_string(a.var));
    return values[a.var];
  };
  auto as_i32 = [&](const Value& v) -> const std::vector<int32_t>& {
    if (v.kind != Value::I32) bail("not an i32");
    return v.i;
  };
  size_t cur = 0, steps = 0;
  while (cur < instrs.size()) {
    if (++steps > (1ull << 32)) bail("interpreter: step limit");
    const ssa::Instr& in = instrs[cur];
    Value value;
    long jump = -1;
    switch (in.op) {
      case UGHIP_I_DEFINE_GLOBAL:
        value.kind = Value::Ptr;
        value.buf = in.n;
        break;
      case UGHIP_I_CONST:
      case UGHIP_I_DEFINE_ACC: value = from_const(in.a); break;
      case UGHIP_I_IF: {
        Value c = get(in.a);
        const auto& cv = as_i32(c);
        bool all_jump = true, any_jump = false;
        for (size_t l = 0; l < N; ++l) {
          if (cv[l] == 0) any_jump = true;
          else all_jump = false;
        }
        if (all_jump != any_jump) bail("diverging threads in warp");
        if (all_jump) {
          values[cur] = Value();
          jump = (long)in.v + 1;
        }
        break;
      }
      case UGHIP_I_RANGE: {
        if (values[cur].kind == Value::None) {
          value = get(in.a);
        } else {
          std::vector<int32_t> nv = as_i32(values[cur]);
          for (auto& x : nv) x += (int32_t)in.n;
          Value up = get(in.b);
          const auto& uv = as_i32(up);
          bool all_jump = true, any_jump = false;
          for (size_t l = 0; l < N; ++l) {
            if (nv[l] >= uv[l]) any_jump = true;
            else all_jump = false;
          }
          if (all_jump != any_jump) bail("diverging threads in warp");
          if (all_jump) {
            values[cur] = Value();  // re-initialise in case the loop is entered again
            jump = (long)in.v + 1;
          } else {
            value.kind = Value::I32;
            value.i = nv;
          }
        }
        break;
      }
      case UGHIP_I_ASSIGN: {
        value = get(in.a);
        values[in.v] = value;
        break;
      }
      case UGHIP_I_END_IF: break;
      case UGHIP_I_END_RANGE: jump = (long)in.v; break;
      case UGHIP_I_LOAD: {
        Value off = get(in.a);
        const auto& ov = as_i32(off);
        const Value& p = values[in.v];
        if (p.kind == Value::Ptr) {
          if (p.buf >= buffers.size()) bail("no buffer for load");
          const InterpBuffer& b = buffers[p.buf];
          if (b.dtype == DType::F32) {
            value.kind = Value::F32;
            value.f.resize(N);
            for (size_t l = 0; l < N; ++l) {
              if (ov[l] < 0 || (size_t)ov[l] >= b.len) bail("load out of bounds");
              value.f[l] = static_cast<const float*>(b.data)[ov[l]];
            }
          } else if (b.dtype == DType::I32) {
            value.kind = Value::I32;
            value.i.resize(N);
            for (size_t l = 0; l < N; ++l) {
              if (ov[l] < 0 || (size_t)ov[l] >= b.len) bail("load out of bounds");
              value.i[l] = static_cast<const int32_t*>(b.data)[ov[l]];
            }
          } else {
            bail("interpreter: unsupported buffer dtype");
          }
        } else if (p.kind == Value::LocalPtr) {
          const Local& b = locals[p.buf];
          if (b.dtype == DType::F32) {
            value.kind = Value::F32;
            value.f.resize(N);
            for (size_t l = 0; l < N; ++l) value.f[l] = b.f.at((size_t)ov[l]);
          } else {
            value.kind = Value::I32;
            value.i.resize(N);
            for (size_t l = 0; l < N; ++l) value.i[l] = b.i.at((size_t)ov[l]);
          }
        } else {
          bail("unexpected dtype for src in load");
        }
        break;
      }
      case UGHIP_I_STORE: {
        Value off = get(in.a);
        const auto& ov = as_i32(off);
        value = get(in.b);
        const Value& p = values[in.v];
        if (p.kind == Value::Ptr) {
          if (p.buf >= buffers.size()) bail("no buffer for store");
          InterpBuffer& b = buffers[p.buf];
          for (size_t l = 0; l < N; ++l) {
            if (ov[l] < 0 || (size_t)ov[l] >= b.len) bail("store out of bounds");
            if (b.dtype == DType::F32 && value.kind == Value::F32) static_cast<float*>(b.data)[ov[l]] = value.f[l];
            else if (b.dtype == DType::I32 && value.kind == Value::I32) static_cast<int32_t*>(b.data)[ov[l]] = value.i[l];
            else bail("unexpected dtype for value in store");
          }
        } else if (p.kind == Value::LocalPtr) {
          Local& b = locals[p.buf];
          for (size_t l = 0; l < N; ++l) {
            if (b.dtype == DType::F32 && value.kind == Value::F32) b.f.at((size_t)ov[l]) = value.f[l];
            else if (b.dtype == DType::I32 && value.kind == Value::I32) b.i.at((size_t)ov[l]) = value.i[l];
            else bail("unexpected dtype for value in store");
          }
        } else {
          bail("unexpected dtype for src in store");
        }
        break;
      }
      case UGHIP_I_BINARY: {
        Value a = get(in.a), b = get(in.b);
        if (a.kind == Value::F32 && b.kind == Value::F32) {
          value.kind = Value::F32;
          value.f.resize(N);
          for (size_t l = 0; l < N; ++l) {
            float x = a.f[l], y = b.f[l], r = 0;
            switch (in.sub) {
              case UGHIP_B_ADD: r = x + y; break;
              case UGHIP_B_SUB: r = x - y; break;
              case UGHIP_B_MUL: r = x * y; break;
              case UGHIP_B_DIV: r = x / y; break;
              case UGHIP_B_MOD: r = std::fmod(x, y); break;
              case UGHIP_B_MIN: r = std::fmin(x, y); break;
              case UGHIP_B_MAX: r = std::fmax(x, y); break;
            }
            value.f[l] = r;
          }
        } else if (a.kind == Value::I32 && b.kind == Value::I32) {
          value.kind = Value::I32;
          value.i.resize(N);
          for (size_t l = 0; l < N; ++l) {
            int32_t x = a.i[l], y = b.i[l], r = 0;
            switch (in.sub) {
              case UGHIP_B_ADD: r = x + y; break;
              case UGHIP_B_SUB: r = x - y; break;
              case UGHIP_B_MUL: r = x * y; break;
              case UGHIP_B_DIV:
                if (y == 0) bail("division by zero");
                r = x / y;
                break;
              case UGHIP_B_MOD:
                if (y == 0) bail("division by zero");
                r = x % y;
                break;
              case UGHIP_B_MIN: r = std::min(x, y); break;
              case UGHIP_B_MAX: r = std::max(x, y); break;
            }
            value.i[l] = r;
          }
        } else {
          bail("dtype mismatch for binary op");
        }
        break;
      }
      case UGHIP_I_UNARY: {
        Value a = get(in.a);
        if (in.sub == UGHIP_U_ID) {
          value = a;
        } else if (in.sub == UGHIP_U_CAST) {
          if (a.kind == Value::F32 && in.dtype == UGHIP_F32) value = a;
          else if (a.kind == Value::I32 && in.dtype == UGHIP_I32) value = a;
          else if (a.kind == Value::F32 && in.dtype == UGHIP_I32) {
            value.kind = Value::I32;
            for (float x : a.f) value.i.push_back((int32_t)x);
          } else if (a.kind == Value::I32 && in.dtype == UGHIP_F32) {
            value.kind = Value::F32;
            for (int32_t x : a.i) value.f.push_back((float)x);
          } else {
            bail("dtype mismatch for cast");
          }
        } else if (a.kind == Value::F32) {
          value.kind = Value::F32;
          for (float x : a.f) {
            float r = 0;
            switch (in.sub) {
              case UGHIP_U_NEG: r = -x; break;
              case UGHIP_U_EXP: r = std::exp(x); break;
              case UGHIP_U_SQRT: r = std::sqrt(x); break;
              case UGHIP_U_SIN: r = std::sin(x); break;
              case UGHIP_U_COS: r = std::cos(x); break;
            }
            value.f.push_back(r);
          }
        } else if (a.kind == Value::I32 && in.sub == UGHIP_U_NEG) {
          value.kind = Value::I32;
          for (int32_t x : a.i) value.i.push_back(-x);
        } else {
          bail("dtype mismatch for unary op");
        }
        break;
      }
      case UGHIP_I_SPECIAL:
        if (in.sub == UGHIP_SPECIAL_THREAD_IDX) {
          value.kind = Value::I32;
          for (size_t l = 0; l < N; ++l) value.i.push_back((int32_t)l);
        } else {
          value = splat_i((int32_t)grid_idx);
        }
        break;
      case UGHIP_I_BARRIER: break;
      case UGHIP_I_REDUCE_LOCAL: {
        Value a = get(in.a);
        if (a.kind == Value::F32) {
          float r = in.sub == UGHIP_R_SUM ? 0.f : (in.sub == UGHIP_R_MAX ? -INFINITY : INFINITY);
          for (float x : a.f) r = in.sub == UGHIP_R_SUM ? r + x : (in.sub == UGHIP_R_MAX ? std::fmax(r, x) : std::fmin(r, x));
          value = splat_f(r);
        } else if (a.kind == Value::I32) {
          int32_t r = in.sub == UGHIP_R_SUM ? 0 : (in.sub == UGHIP_R_MAX ? INT32_MIN : INT32_MAX);
          for (int32_t x : a.i) r = in.sub == UGHIP_R_SUM ? r + x : (in.sub == UGHIP_R_MAX ? std::max(r, x) : std::min(r, x));
          value = splat_i(r);
        } else {
          bail("dtype mismatch for reduce-local");
        }
        break;
      }
      case UGHIP_I_DEFINE_LOCAL: {
        Local l;
        l.dtype = (DType)in.dtype;
        if (l.dtype == DType::F32) l.f.assign(in.n, 0.f);
        else if (l.dtype == DType::I32) l.i.assign(in.n, 0);
        else bail("interpreter: unsupported local dtype");
        value.kind = Value::LocalPtr;
        value.buf = locals.size();
        locals.push_back(std::move(l));
        break;
      }
      default: bail("interpreter: unknown instruction");
    }
    if (value.kind != Value::None) values[cur] = value;
    cur = jump >= 0 ? (size_t)jump : cur + 1;
  }
}

}  // namespace ug_oracle
