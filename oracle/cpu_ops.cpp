// ORACLE -- TEST INFRASTRUCTURE ONLY.
// ug-llama's five custom ops on the CPU: restatement of ug-llama/src/cpu_ops.rs:6-167 (f32 only,
// same loop order and the same sequential f32 sums), plus the C entry points the tests load.
// Pinned by: invariants in the GPU suite (pair norms, identity at position 0, idempotent mask,
// cat == concatenate, softmax against f64) and, through the whole model, by an independent float64
// numpy llama (tests/test_llama_numpy_reference.py).  No reference fixture holds outputs of these
// ops, so parity with the reference's own binaries is unpinned.
#include <cmath>
#include <cstring>

#include "oracle.h"

namespace ug_oracle {

using namespace ug;
using ug_llama::LB;

namespace {

float* f32_mut(Slice* s) {
  CpuSlice& c = cpu_slice(*s);
  if (c.dtype() != DType::F32) bail(std::string("unexpected dtype, expected F32, got ") + dtype_str(c.dtype()));
  return reinterpret_cast<float*>(c.data());
}
const float* f32(Slice* s) { return f32_mut(s); }
const int32_t* i32(Slice* s) {
  CpuSlice& c = cpu_slice(*s);
  if (c.dtype() != DType::I32) bail(std::string("unexpected dtype, expected I32, got ") + dtype_str(c.dtype()));
  return reinterpret_cast<const int32_t*>(c.data());
}

struct CpuOps : ug_llama::Ops {
  // cpu_ops.rs:6-31
  LB custom_softmax(const LB& src) const override {
    size_t dim_m1 = src.dims()[src.rank() - 1];
    auto f = [dim_m1](const std::vector<Slice*>& vs) {
      if (vs.size() != 2) bail("softmax: expected 2 slices");
      const float* s = f32(vs[0]);
      float* d = f32_mut(vs[1]);
      size_t n = vs[0]->len();
      for (size_t r = 0; dim_m1 && r + dim_m1 <= n; r += dim_m1) {
        float mx = -INFINITY;
        for (size_t j = 0; j < dim_m1; ++j) mx = std::fmax(s[r + j], mx);
        for (size_t j = 0; j < dim_m1; ++j) d[r + j] = std::exp(s[r + j] - mx);
        float sum = 0.f;
        for (size_t j = 0; j < dim_m1; ++j) sum += d[r + j];
        for (size_t j = 0; j < dim_m1; ++j) d[r + j] /= sum;
      }
    };
    return LB::custom(f, {src}, src.shape(), src.dtype(), src.device());
  }

  // cpu_ops.rs:33-56
  LB causal_mask(const LB& src) const override {
    if (src.rank() != 4) bail("causal_mask: expected a rank-4 tensor");
    size_t s1 = src.dims()[2], s2 = src.dims()[3];
    auto f = [s1, s2](const std::vector<Slice*>& vs) {
      if (vs.size() != 2) bail("causal_mask: expected 2 slices");
      const float* s = f32(vs[0]);
      float* d = f32_mut(vs[1]);
      size_t n = vs[0]->len(), chunk = s1 * s2;
      for (size_t c = 0; chunk && c + chunk <= n; c += chunk)
        for (size_t i1 = 0; i1 < s1; ++i1) {
          for (size_t i2 = 0; i2 <= i1 && i2 < s2; ++i2) d[c + i1 * s2 + i2] = s[c + i1 * s2 + i2];
          for (size_t i2 = i1 + 1; i2 < s2; ++i2) d[c + i1 * s2 + i2] = -INFINITY;
        }
    };
    return LB::custom(f, {src}, src.shape(), src.dtype(), src.device());
  }

  // cpu_ops.rs:58-89
  LB rope_i(const LB& src, const LB& cos, const LB& sin, const LB& pos) const override {
    if (src.rank() != 4) bail("rope_i: expected a rank-4 tensor");
    size_t t = src.dims()[2], d = src.dims()[3];
    auto f = [t, d](const std::vector<Slice*>& vs) {
      if (vs.size() != 5) bail("rope_i: expected 5 slices");
      const float* s = f32(vs[0]);
      const float* c = f32(vs[1]);
      const float* sn = f32(vs[2]);
      size_t p = (size_t)i32(vs[3])[0];
      float* o = f32_mut(vs[4]);
      size_t n = vs[0]->len(), chunk = t * d;
      if (p * d / 2 + chunk / 2 > vs[1]->len() || p * d / 2 + chunk / 2 > vs[2]->len()) bail("rope_i: position out of range of the cos/sin tables");
      c += p * d / 2;
      sn += p * d / 2;
      for (size_t b = 0; chunk && b + chunk <= n; b += chunk)
        for (size_t i2 = 0; i2 < chunk / 2; ++i2) {
          size_t i = 2 * i2;
          float a = s[b + i], bb = s[b + i + 1];
          o[b + i] = a * c[i2] - bb * sn[i2];
          o[b + i + 1] = a * sn[i2] + bb * c[i2];
        }
    };
    return LB::custom(f, {src, cos, sin, pos}, src.shape(), src.dtype(), src.device());
  }

  // cpu_ops.rs:91-126
  LB rope(const LB& src, const LB& cos, const LB& sin, const LB& pos) const override {
    if (src.rank() != 4) bail("rope: expected a rank-4 tensor");
    size_t t = src.dims()[2], d = src.dims()[3];
    auto f = [t, d](const std::vector<Slice*>& vs) {
      if (vs.size() != 5) bail("rope: expected 5 slices");
      const float* s = f32(vs[0]);
      const float* c = f32(vs[1]);
      const float* sn = f32(vs[2]);
      size_t p = (size_t)i32(vs[3])[0];
      float* o = f32_mut(vs[4]);
      size_t n = vs[0]->len(), chunk = t * d;
      if (p * d / 2 + chunk / 2 > vs[1]->len() || p * d / 2 + chunk / 2 > vs[2]->len()) bail("rope: position out of range of the cos/sin tables");
      c += p * d / 2;
      sn += p * d / 2;
      for (size_t b = 0; chunk && b + chunk <= n; b += chunk)
        for (size_t i_t = 0; i_t < t; ++i_t)
          for (size_t i_d = 0; i_d < d / 2; ++i_d) {
            size_t i1 = i_t * d + i_d, i2 = i1 + d / 2, ics = i_t * (d / 2) + i_d;
            float x1 = s[b + i1], x2 = s[b + i2];
            o[b + i1] = x1 * c[ics] - x2 * sn[ics];
            o[b + i2] = x1 * sn[ics] + x2 * c[ics];
          }
    };
    return LB::custom(f, {src, cos, sin, pos}, src.shape(), src.dtype(), src.device());
  }

  // cpu_ops.rs:128-167
  LB cat(const LB& lhs, const LB& rhs, size_t axis) const override {
    const auto& ld = lhs.dims();
    const auto& rd = rhs.dims();
    if (axis >= ld.size()) bail("unexpected axis " + std::to_string(axis) + " for cat " + lhs.shape().str());
    if (ld.size() != rd.size()) bail("unexpected shapes for cat " + lhs.shape().str() + " " + rhs.shape().str());
    for (size_t i = 0; i < ld.size(); ++i)
      if (i != axis && ld[i] != rd[i]) bail("unexpected shapes for cat " + lhs.shape().str() + " " + rhs.shape().str());
    std::vector<size_t> dd = ld;
    dd[axis] = ld[axis] + rd[axis];
    size_t d1 = 1, d2_l = 1, d2_r = 1;
    for (size_t i = 0; i < axis; ++i) d1 *= ld[i];
    for (size_t i = axis; i < ld.size(); ++i) {
      d2_l *= ld[i];
      d2_r *= rd[i];
    }
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 3) bail("cat: expected 3 slices");
      const float* l = f32(vs[0]);
      const float* r = f32(vs[1]);
      float* o = f32_mut(vs[2]);
      size_t d2 = d2_l + d2_r;
      for (size_t i1 = 0; i1 < d1; ++i1) {
        if (d2_l) std::memcpy(o + i1 * d2, l + i1 * d2_l, d2_l * sizeof(float));
        if (d2_r) std::memcpy(o + i1 * d2 + d2_l, r + i1 * d2_r, d2_r * sizeof(float));
      }
    };
    return LB::custom(f, {lhs, rhs}, Shape(dd), lhs.dtype(), lhs.device());
  }
};

thread_local std::string g_err;
template <typename F>
int guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_err = e.what();
    return 1;
  }
}

}  // namespace

std::shared_ptr<ug_llama::Ops> cpu_ops() { return std::make_shared<CpuOps>(); }

}  // namespace ug_oracle

// ---- C entry points for the tests (handles are interchangeable with libug_host's) --------------------
using namespace ug_oracle;

extern "C" {

const char* ugo_last_error(void) { return g_err.c_str(); }

int ugo_cpu_device_new(void** out) {
  return guard([&] { *out = new ug::DevicePtr(std::make_shared<CpuDevice>()); });
}

int ugo_llama_ops_cpu(void** out) {
  return guard([&] { *out = new std::shared_ptr<ug_llama::Ops>(cpu_ops()); });
}

// C text the CPU backend would hand to gcc for `kernel`.
int ugo_gen_c(void* kernel, const char* func_name, char* buf, size_t buf_len, size_t* out_len) {
  return guard([&] {
    std::string s = gen_c(func_name, *static_cast<ug::ssa::Kernel*>(kernel));
    if (out_len) *out_len = s.size();
    if (buf && buf_len) {
      size_t n = std::min(buf_len - 1, s.size());
      std::memcpy(buf, s.data(), n);
      buf[n] = 0;
    }
  });
}

// CpuDevice::compile_c (ug-core/tests/cpu_tests.rs): compile literal C text.
int ugo_compile_c(void* dev, const char* c_code, const char* func_name, void** out_func) {
  return guard([&] {
    CpuDevice* d = dynamic_cast<CpuDevice*>(static_cast<ug::DevicePtr*>(dev)->get());
    if (!d) ug::bail("not a cpu device");
    *out_func = new std::shared_ptr<ug::Func>(d->compile_c(c_code, func_name));
  });
}

// interpreter::eval_ssa::<N>(kernel, buffers, &[], grid_idx)
int ugo_eval_ssa(void* kernel, void** datas, const int* dtypes, const size_t* lens, size_t n_buffers, size_t n_lanes, size_t grid_idx) {
  return guard([&] {
    std::vector<InterpBuffer> bufs;
    for (size_t i = 0; i < n_buffers; ++i) bufs.push_back(InterpBuffer{(ug::DType)dtypes[i], datas[i], lens[i]});
    eval_ssa(*static_cast<ug::ssa::Kernel*>(kernel), bufs, n_lanes, grid_idx);
  });
}

}  // extern "C"
