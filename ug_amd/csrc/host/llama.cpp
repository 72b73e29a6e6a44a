// Llama graph over ug::LazyBuffer.  Mirrors ug-llama/src/model.rs op for op, so the kernels
// a device sees (names, shapes, argument order) are those of the reference.
#include "llama.h"

#include <atomic>
#include <mutex>
#include <chrono>
#include <cmath>
#include <thread>

#include "hip_device.h"
#include "rng.h"
#include "ug/block.h"
#include "ug/safetensors.h"

namespace ug_llama {

namespace {
const char* const kSwitchNames[SW_COUNT] = {"NO_FOLD_EPILOGUES", "NO_APPEND_PAIR", "VERBOSE", "NO_LAYER_STEPS", "HOST_ARGMAX", "NO_OVERLAP"};
std::atomic<int> g_switch[SW_COUNT];
std::once_flag g_switch_once;
void switches_init() {
  std::call_once(g_switch_once, [] {
    for (int i = 0; i < SW_COUNT; ++i) g_switch[i].store(getenv((std::string("UG_LLAMA_") + kSwitchNames[i]).c_str()) != nullptr, std::memory_order_relaxed);
  });
}
}  // namespace
bool switch_on(Switch s) {
  switches_init();
  return g_switch[s].load(std::memory_order_relaxed) != 0;
}
bool set_switch(const std::string& name, bool on) {
  switches_init();
  const std::string n = name.rfind("UG_LLAMA_", 0) == 0 ? name.substr(9) : name;
  for (int i = 0; i < SW_COUNT; ++i)
    if (n == kSwitchNames[i]) {
      g_switch[i].store(on, std::memory_order_relaxed);
      return true;
    }
  return false;
}


using namespace ug;

// ---- HIP custom ops (counterpart of ug-llama/src/cuda_ops.rs:17-179) -------------------------
namespace {

void hip_check(int rc, const char* what) {
  if (rc) bail(std::string(what) + ": " + ughip_last_error());
}

ughip_device* hip_dev(const LB& lb) {
  HipDevice* d = dynamic_cast<HipDevice*>(lb.device().get());
  if (!d) bail("hip custom op used with a non-hip device");
  return d->raw();
}

struct HipOps : Ops {
  explicit HipOps(bool bf16x3 = false) : bf16x3_(bf16x3) {}
  bool bf16x3_;

  LB rope_any(const LB& src, const LB& cos, const LB& sin, const LB& pos, int interleaved) const {
    if (src.rank() != 4) bail("rope: expected a rank-4 tensor, got " + src.shape().str());
    size_t b = src.dims()[0], h = src.dims()[1], t = src.dims()[2], d = src.dims()[3];
    ughip_device* dev = hip_dev(src);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 5) bail("rope: expected 5 slices");
      hip_check(ughip_rope(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), hip_raw_slice(*vs[3]), hip_raw_slice(*vs[4]),
                           b * h, t, d, interleaved),
                "rope");
    };
    return LB::custom(f, {src, cos, sin, pos}, src.shape(), src.dtype(), src.device());
  }
  LB rope_i(const LB& src, const LB& cos, const LB& sin, const LB& pos) const override { return rope_any(src, cos, sin, pos, 1); }
  LB rope(const LB& src, const LB& cos, const LB& sin, const LB& pos) const override { return rope_any(src, cos, sin, pos, 0); }

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
    ughip_device* dev = hip_dev(lhs);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 3) bail("cat: expected 3 slices");
      hip_check(ughip_cat(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), d1, d2_l, d2_r), "cat");
    };
    return LB::custom(f, {lhs, rhs}, Shape(dd), lhs.dtype(), lhs.device());
  }

  LB custom_softmax(const LB& src) const override {
    size_t dim_m1 = src.dims()[src.rank() - 1];
    size_t rows = dim_m1 ? src.elem_count() / dim_m1 : 0;
    ughip_device* dev = hip_dev(src);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 2) bail("softmax: expected 2 slices");
      hip_check(ughip_softmax_rows(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), rows, dim_m1), "custom_softmax");
    };
    return LB::custom(f, {src}, src.shape(), src.dtype(), src.device());
  }

  LB causal_softmax(const LB& att) const override {
    if (att.rank() != 4) bail("causal_softmax: expected a rank-4 tensor, got " + att.shape().str());
    size_t bh = att.dims()[0] * att.dims()[1], s1 = att.dims()[2], s2 = att.dims()[3];
    ughip_device* dev = hip_dev(att);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 2) bail("causal_softmax: expected 2 slices");
      hip_check(ughip_causal_softmax_rows(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), bh, s1, s2), "causal_softmax");
    };
    return LB::custom(f, {att}, att.shape(), att.dtype(), att.device());
  }

  LB attention_decode(const LB& q, const LB& k, const LB& v, float scale) const override {
    if (q.rank() != 4 || k.rank() != 4 || v.rank() != 4 || q.dims()[2] != 1) bail("attention_decode: expected q [b, nh, 1, d] and k, v [b, nkv, s, d]");
    size_t b = q.dims()[0], nh = q.dims()[1], d = q.dims()[3], nkv = k.dims()[1], s = k.dims()[2];
    if (k.dims() != v.dims() || k.dims()[0] != b || k.dims()[3] != d) bail("attention_decode: mismatched shapes " + q.shape().str() + " " + k.shape().str());
    ughip_device* dev = hip_dev(q);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 4) bail("attention_decode: expected 4 slices");
      hip_check(ughip_attention_decode(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), hip_raw_slice(*vs[3]), b, nh, nkv, s, d, scale),
                "attention_decode");
    };
    return LB::custom(f, {q, k, v}, q.shape(), q.dtype(), q.device());
  }

  LB rope_append(const LB& cache, const LB& x, const LB* cos, const LB* sin, const LB* pos, bool interleaved) const override {
    if (cache.rank() != 4 || x.rank() != 3 || x.dims()[1] != 1) bail("rope_append: expected cache [b, n, s, d] and x [b, 1, n * d]");
    size_t b = cache.dims()[0], n = cache.dims()[1], s_old = cache.dims()[2], d = cache.dims()[3];
    if (x.dims()[0] != b || x.dims()[2] != n * d) bail("rope_append: mismatched shapes " + cache.shape().str() + " " + x.shape().str());
    if (d % 8 != 0) return Ops::rope_append(cache, x, cos, sin, pos, interleaved);
    ughip_device* dev = hip_dev(x);
    const bool with_rope = cos != nullptr;
    int il = interleaved ? 1 : 0;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 6u : 3u)) bail("rope_append: unexpected number of slices");
      ughip_slice* dst = hip_raw_slice(*vs.back());
      hip_check(ughip_rope_append(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), dst, b * n, s_old, d, with_rope ? hip_raw_slice(*vs[2]) : nullptr,
                                  with_rope ? hip_raw_slice(*vs[3]) : nullptr, with_rope ? hip_raw_slice(*vs[4]) : nullptr, il),
                "rope_append");
    };
    std::vector<LB> args = {cache, x};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return LB::custom(f, args, Shape({b, n, s_old + 1, d}), x.dtype(), x.device());
  }

  LB attention_decode_flat(const LB& q, const LB& k, const LB& v, float scale, const LB* cos, const LB* sin, const LB* pos, bool interleaved) const override {
    if (q.rank() != 3 || q.dims()[1] != 1 || k.rank() != 4 || v.rank() != 4) bail("attention_decode_flat: expected q [b, 1, nh * d] and k, v [b, nkv, s, d]");
    size_t b = q.dims()[0], nkv = k.dims()[1], s = k.dims()[2], d = k.dims()[3];
    if (k.dims() != v.dims() || k.dims()[0] != b || d == 0 || q.dims()[2] % d != 0)
      bail("attention_decode_flat: mismatched shapes " + q.shape().str() + " " + k.shape().str());
    size_t nh = q.dims()[2] / d;
    ughip_device* dev = hip_dev(q);
    const bool with_rope = cos != nullptr;
    int il = interleaved ? 1 : 0;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 7u : 4u)) bail("attention_decode_flat: unexpected number of slices");
      ughip_slice* dst = hip_raw_slice(*vs.back());
      hip_check(ughip_attention_decode_rope(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), dst, b, nh, nkv, s, d, scale,
                                            with_rope ? hip_raw_slice(*vs[3]) : nullptr, with_rope ? hip_raw_slice(*vs[4]) : nullptr,
                                            with_rope ? hip_raw_slice(*vs[5]) : nullptr, il),
                "attention_decode_flat");
    };
    std::vector<LB> args = {q, k, v};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return LB::custom(f, args, q.shape(), q.dtype(), q.device());
  }

  LB causal_mask(const LB& src) const override {
    if (src.rank() != 4) bail("causal_mask: expected a rank-4 tensor, got " + src.shape().str());
    size_t bh = src.dims()[0] * src.dims()[1], s1 = src.dims()[2], s2 = src.dims()[3];
    ughip_device* dev = hip_dev(src);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 2) bail("causal_mask: expected 2 slices");
      hip_check(ughip_causal_mask(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), bh, s1, s2), "causal_mask");
    };
    return LB::custom(f, {src}, src.shape(), src.dtype(), src.device());
  }

  // head sizes attention_cached has kernels for at any number of query positions
  size_t kv_cache_capacity(size_t max_positions, size_t head_dim) const override {
    return head_dim == 32 || head_dim == 64 || head_dim == 128 ? max_positions : 0;
  }

  bool packed_projections() const override { return true; }

  LB kv_append(const LB& cache, size_t len, const LB& x, const LB* cos, const LB* sin, const LB* pos, bool interleaved, size_t x_offset,
               size_t x_row_stride) const override {
    if (cache.rank() != 4 || x.rank() != 3) bail("kv_append: expected cache [b, n, cap, d] and x [b, t, n * d]");
    size_t b = cache.dims()[0], n = cache.dims()[1], cap = cache.dims()[2], d = cache.dims()[3], t = x.dims()[1];
    const bool packed = x_offset != 0 || x_row_stride != 0;
    if (x.dims()[0] != b || (packed ? x_row_stride != x.dims()[2] || x_offset + n * d > x_row_stride : x.dims()[2] != n * d))
      bail("kv_append: mismatched shapes " + cache.shape().str() + " " + x.shape().str());
    // a cache with exactly the rows written so far is the reference's growing representation (model.rs:226-230);
    // one that was preallocated and is full is refused below, not quietly reallocated
    if (cap == len || d % 4 != 0) return Ops::kv_append(cache, len, x, cos, sin, pos, interleaved, x_offset, x_row_stride);
    if (len + t > cap) bail("kv_append: " + std::to_string(len + t) + " rows exceed the cache capacity " + std::to_string(cap));
    ughip_device* dev = hip_dev(x);
    const bool with_rope = cos != nullptr;
    int il = interleaved ? 1 : 0;
    // in-place op: arguments first, the cache last (schedule.rs:404-413)
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 5u : 2u)) bail("kv_append: unexpected number of slices");
      hip_check(ughip_kv_append(dev, hip_raw_slice(*vs.back()), hip_raw_slice(*vs[0]), x_offset, x_row_stride, b, n, cap, len, t, d,
                                with_rope ? hip_raw_slice(*vs[1]) : nullptr,
                                with_rope ? hip_raw_slice(*vs[2]) : nullptr, with_rope ? hip_raw_slice(*vs[3]) : nullptr, il),
                "kv_append");
    };
    std::vector<LB> args = {x};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return cache.custom_ip(f, args);
  }

  LB attention_cached(const LB& q, const LB& k, const LB& v, size_t s, float scale, const LB* cos, const LB* sin, const LB* pos, bool interleaved,
                      size_t q_offset, size_t q_row_stride, size_t n_heads) const override {
    if (q.rank() != 3 || k.rank() != 4 || v.rank() != 4) bail("attention_cached: expected q [b, t, nh * d] and k, v [b, nkv, cap, d]");
    size_t b = q.dims()[0], t = q.dims()[1], nkv = k.dims()[1], cap = k.dims()[2], d = k.dims()[3];
    const bool packed = q_offset != 0 || q_row_stride != 0;
    if (k.dims() != v.dims() || k.dims()[0] != b || d == 0 || s > cap || t > s || (packed ? n_heads == 0 || q_row_stride != q.dims()[2] || q_offset + n_heads * d > q_row_stride
                                                                                              : q.dims()[2] % d != 0 || (n_heads != 0 && n_heads * d != q.dims()[2])))
      bail("attention_cached: mismatched shapes " + q.shape().str() + " " + k.shape().str() + " with " + std::to_string(s) + " keys");
    size_t nh = packed ? n_heads : q.dims()[2] / d;
    const bool one = t == 1 && d >= 16 && d <= 256 && (d & (d - 1)) == 0;
    const bool many = t > 1 && (d == 32 || d == 64 || d == 128);
    if (!one && !many) return Ops::attention_cached(q, k, v, s, scale, cos, sin, pos, interleaved, q_offset, q_row_stride, n_heads);
    ughip_device* dev = hip_dev(q);
    const bool with_rope = cos != nullptr;
    int il = interleaved ? 1 : 0;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 7u : 4u)) bail("attention_cached: unexpected number of slices");
      ughip_slice* dst = hip_raw_slice(*vs.back());
      hip_check(ughip_attention_cached(dev, hip_raw_slice(*vs[0]), q_offset, q_row_stride, hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), dst, b, nh, nkv, t, s, cap, d, scale,
                                       with_rope ? hip_raw_slice(*vs[3]) : nullptr, with_rope ? hip_raw_slice(*vs[4]) : nullptr,
                                       with_rope ? hip_raw_slice(*vs[5]) : nullptr, il),
                "attention_cached");
    };
    std::vector<LB> args = {q, k, v};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return LB::custom(f, args, Shape({b, t, nh * d}), q.dtype(), q.device());
  }

  // One input row of f32 against row-major [n, k] matrices stored as f32 or bf16 (all alike): the
  // shapes the fused GEMV kernels take.
  static bool one_f32_row(const LB& x, const std::vector<const LB*>& ws) {
    if (x.rank() != 3 || x.dims()[0] * x.dims()[1] != 1 || x.dtype() != DType::F32 || x.dims()[2] % 4 != 0) return false;
    for (const LB* w : ws) {
      if (w->rank() != 2 || w->dims()[1] != x.dims()[2] || w->dtype() != ws[0]->dtype()) return false;
      if (w->dtype() != DType::F32 && w->dtype() != DType::BF16) return false;
    }
    return true;
  }

  // the fused norm keeps the row in registers
  static bool rms_ok(const LB& x, const LB* alpha) {
    return !alpha || (x.dims()[2] <= 4096 && alpha->dtype() == DType::F32 && alpha->elem_count() == x.dims()[2]);
  }

  // f32 rows against a matrix stored as bf16: one row is a fused projection without neighbours; from 9
  // rows up (where an f32 matrix takes the tiled kernel too) ughip_matmul reads the matrix as it is;
  // the row counts in between and the shapes no tile divides widen it first.  Each way the numbers
  // are those of the f32 matrix with the same values.
  LB linear(const LB& x, const LB& w) const override {
    const size_t rows = x.rank() ? x.elem_count() / x.dims().back() : 0;
    if (x.dtype() == DType::F32 && w.dtype() == DType::BF16 && rows == 1 && x.rank() == 3 && one_f32_row(x, {&w})) return linear_packed(x, {w}, nullptr, 0.f);
    if (x.dtype() != DType::F32 || w.dtype() != DType::BF16 || w.rank() != 2 || x.rank() < 2 || w.dims()[1] != x.dims().back() || rows <= 1 ||
        w.dims()[1] % 32 != 0)
      return Ops::linear(x, w);
    const size_t n = w.dims()[0], k = w.dims()[1];
    ughip_device* dev = hip_dev(x);
    const bool x3 = product_for(w, k, rows) == UGHIP_PRODUCT_BF16X3 && n % 8 == 0;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 3) bail("linear: expected 3 slices");
      if (x3) {
        hip_check(ughip_linear_rows(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), rows, n, k, UGHIP_PRODUCT_BF16X3), "linear");
        return;
      }
      const size_t ld[3] = {1, rows, k}, ls[3] = {rows * k, k, 1}, rd[3] = {1, k, n}, rs[3] = {n * k, 1, k};
      hip_check(ughip_matmul(dev, hip_raw_slice(*vs[2]), hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), 1, rows, n, k, 3, ld, ls, 0, rd, rs, 0), "linear");
    };
    std::vector<size_t> dims = x.dims();
    dims.back() = n;
    return LB::custom(f, {x, w}, Shape(dims), DType::F32, x.device());
  }

  LB linear_packed(const LB& x, const std::vector<LB>& ws, const LB* alpha, float eps) const override {
    std::vector<const LB*> wp;
    for (const LB& w : ws) wp.push_back(&w);
    if (ws.empty() || ws.size() > 3 || !one_f32_row(x, wp) || !rms_ok(x, alpha)) return Ops::linear_packed(x, ws, alpha, eps);
    std::vector<size_t> ns;
    size_t total = 0, k = x.dims()[2];
    for (const LB& w : ws) {
      ns.push_back(w.dims()[0]);
      total += w.dims()[0];
    }
    ughip_device* dev = hip_dev(x);
    size_t n_mats = ws.size();
    const bool norm = alpha != nullptr;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != n_mats + 2 + (norm ? 1 : 0)) bail("linear_packed: unexpected number of slices");
      const ughip_slice* w[3] = {nullptr, nullptr, nullptr};
      for (size_t i = 0; i < n_mats; ++i) w[i] = hip_raw_slice(*vs[1 + i]);
      hip_check(ughip_rms_gemv_multi(dev, hip_raw_slice(*vs[0]), norm ? hip_raw_slice(*vs[1 + n_mats]) : nullptr, eps, n_mats, w, ns.data(), k,
                                     hip_raw_slice(*vs.back())),
                "linear_packed");
    };
    std::vector<LB> args = {x};
    for (const LB& w : ws) args.push_back(w);
    if (norm) args.push_back(*alpha);
    return LB::custom(f, args, Shape({1, 1, total}), x.dtype(), x.device());
  }

  LB gate_up(const LB& x, const LB& w_gate, const LB& w_up, const LB* alpha, float eps) const override {
    if (!one_f32_row(x, {&w_gate, &w_up}) || w_gate.dims() != w_up.dims() || !rms_ok(x, alpha)) return Ops::gate_up(x, w_gate, w_up, alpha, eps);
    size_t n = w_gate.dims()[0], k = x.dims()[2];
    ughip_device* dev = hip_dev(x);
    const bool norm = alpha != nullptr;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (norm ? 5u : 4u)) bail("gate_up: unexpected number of slices");
      hip_check(ughip_rms_gemv_gate_up(dev, hip_raw_slice(*vs[0]), norm ? hip_raw_slice(*vs[3]) : nullptr, eps, hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]),
                                       hip_raw_slice(*vs.back()), n, k),
                "gate_up");
    };
    std::vector<LB> args = {x, w_gate, w_up};
    if (norm) args.push_back(*alpha);
    return LB::custom(f, args, Shape({1, 1, n}), x.dtype(), x.device());
  }

  // How nine or more f32 rows meet this matrix: three bf16 terms per row element on the bf16 matrix pipe when that was
  // asked for and the matrix is bf16 with k a multiple of 64, else the f32 pipe.
  // Up to 32 rows the f32 pipe on a 32-row tile is faster (2.0-2.1 ms for a prompt of 9 .. 32 tokens against 2.3); from 33
  // rows the product that splits the rows itself is (2.30-2.39 ms for 40 .. 64 tokens against 2.50-2.57).
  int product_for(const LB& w, size_t k, size_t rows) const {
    return bf16x3_ && rows > 32 && w.dtype() == DType::BF16 && k % 64 == 0 ? UGHIP_PRODUCT_BF16X3 : UGHIP_PRODUCT_F32;
  }

  // Several positions of f32 rows against a row-major [n, k] matrix (f32 or bf16) in shapes the tiled kernel takes:
  // the fold of its partial tiles can apply the neighbouring op.
  static bool many_f32_rows(const LB& x, const LB& w, size_t n_multiple) {
    if (x.rank() < 2 || w.rank() != 2 || x.dtype() != DType::F32 || (w.dtype() != DType::F32 && w.dtype() != DType::BF16)) return false;
    const size_t k = x.dims().back(), rows = x.elem_count() / (k ? k : 1);
    // 2 .. 8 rows against an F32 matrix take the row-vector kernels; a BF16 matrix would have to be widened for those
    // (three times its bytes moved), so it goes to the tiled product from 2 rows on
    return k != 0 && w.dims()[1] == k && rows >= (w.dtype() == DType::BF16 ? 2u : 9u) && k % 32 == 0 && w.dims()[0] % n_multiple == 0;
  }

  LB gate_up_stacked(const LB& x, const LB& w) const override {
    if (!many_f32_rows(x, w, 16) || switch_on(SW_NO_FOLD_EPILOGUES)) return Ops::gate_up_stacked(x, w);
    const size_t k = x.dims().back(), rows = x.elem_count() / k, n = w.dims()[0] / 2;
    ughip_device* dev = hip_dev(x);
    const int product = product_for(w, k, rows);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 3) bail("gate_up_stacked: expected 3 slices");
      hip_check(ughip_linear_swiglu_rows(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), rows, n, k, product), "gate_up_stacked");
    };
    std::vector<size_t> dims = x.dims();
    dims.back() = n;
    return LB::custom(f, {x, w}, Shape(dims), DType::F32, x.device());
  }

  LB linear_add(const LB& x, const LB& w, const LB& residual) const override {
    if (many_f32_rows(x, w, 8) && residual.dtype() == DType::F32 && residual.elem_count() == x.elem_count() / x.dims().back() * w.dims()[0] &&
        !switch_on(SW_NO_FOLD_EPILOGUES)) {
      const size_t k = x.dims().back(), rows = x.elem_count() / k, n = w.dims()[0];
      ughip_device* dev = hip_dev(x);
      const int product = product_for(w, k, rows);
      auto f = [=](const std::vector<Slice*>& vs) {
        if (vs.size() != 4) bail("linear_add: expected 4 slices");
        hip_check(ughip_linear_add_rows(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), hip_raw_slice(*vs[3]), rows, n, k, product), "linear_add");
      };
      return LB::custom(f, {x, w, residual}, residual.shape(), DType::F32, x.device());
    }
    if (!one_f32_row(x, {&w}) || residual.dtype() != DType::F32 || residual.elem_count() != w.dims()[0]) return Ops::linear_add(x, w, residual);
    size_t n = w.dims()[0], k = x.dims()[2];
    ughip_device* dev = hip_dev(x);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 4) bail("linear_add: expected 4 slices");
      hip_check(ughip_gemv_add(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), hip_raw_slice(*vs[3]), n, k), "linear_add");
    };
    return LB::custom(f, {x, w, residual}, residual.shape(), x.dtype(), x.device());
  }

  // The norm in front of a product of many rows, and the MLP block whole: one schedule item each, and where the
  // three-term product reads planes the passes that write them do the norm / come out of the SwiGLU fold.
  LB linear_norm(const LB& x, const LB& alpha, float eps, const LB& w) const override {
    if (!many_f32_rows(x, w, 8) || alpha.dtype() != DType::F32 || alpha.elem_count() != x.dims().back() || switch_on(SW_NO_FOLD_EPILOGUES))
      return Ops::linear_norm(x, alpha, eps, w);
    const size_t k = x.dims().back(), rows = x.elem_count() / k, n = w.dims()[0];
    ughip_device* dev = hip_dev(x);
    const int product = product_for(w, k, rows);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 4) bail("linear_norm: expected 4 slices");
      hip_check(ughip_rms_linear_rows(dev, hip_raw_slice(*vs[0]), hip_raw_slice(*vs[1]), eps, hip_raw_slice(*vs[2]), hip_raw_slice(*vs[3]), rows, n, k, product), "linear_norm");
    };
    std::vector<size_t> dims = x.dims();
    dims.back() = n;
    return LB::custom(f, {x, alpha, w}, Shape(dims), DType::F32, x.device());
  }

  LB mlp_stacked(const LB& x, const LB* alpha, float eps, const LB& w_gate_up, const LB& w_down, const LB& residual) const override {
    const size_t k = x.rank() ? x.dims().back() : 0, inter = w_gate_up.rank() == 2 ? w_gate_up.dims()[0] / 2 : 0;
    if (!many_f32_rows(x, w_gate_up, 16) || w_down.rank() != 2 || w_down.dtype() != w_gate_up.dtype() || w_down.dims()[1] != inter || inter % 32 != 0 ||
        w_down.dims()[0] % 8 != 0 || residual.dtype() != DType::F32 || residual.elem_count() != x.elem_count() / k * w_down.dims()[0] ||
        (alpha && (alpha->dtype() != DType::F32 || alpha->elem_count() != k)) || switch_on(SW_NO_FOLD_EPILOGUES))
      return Ops::mlp_stacked(x, alpha, eps, w_gate_up, w_down, residual);
    const size_t rows = x.elem_count() / k, n = w_down.dims()[0];
    ughip_device* dev = hip_dev(x);
    // one choice for both products, the one the pieces would make for the first (the second has the longer k)
    const int product = product_for(w_gate_up, k, rows) == UGHIP_PRODUCT_BF16X3 && product_for(w_down, inter, rows) == UGHIP_PRODUCT_BF16X3 ? UGHIP_PRODUCT_BF16X3
                                                                                                                                        : UGHIP_PRODUCT_F32;
    const bool norm = alpha != nullptr;
    // with the norm folded in, the rows and the residual are usually one buffer: a schedule item names a buffer once
    const bool same = x.data().get() == residual.data().get();
    const size_t n_args = 4 + (same ? 0 : 1) + (norm ? 1 : 0);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != n_args) bail("mlp_stacked: unexpected number of slices");
      hip_check(ughip_rms_mlp_rows(dev, hip_raw_slice(*vs[0]), norm ? hip_raw_slice(*vs[n_args - 2]) : nullptr, eps, hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]),
                                   hip_raw_slice(*vs[same ? 0 : 3]), hip_raw_slice(*vs.back()), rows, n, inter, k, product),
                "mlp_stacked");
    };
    std::vector<LB> args = {x, w_gate_up, w_down};
    if (!same) args.push_back(residual);
    if (norm) args.push_back(*alpha);
    return LB::custom(f, args, residual.shape(), DType::F32, x.device());
  }

  LB attention_step(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin, const LB* pos,
                    bool interleaved) const override {
    if (qkv.rank() != 3 || qkv.dims()[1] != 1 || kcache.rank() != 4 || kcache.dims() != vcache.dims()) bail("attention_step: expected qkv [b, 1, row] and caches [b, nkv, cap, d]");
    size_t b = qkv.dims()[0], row = qkv.dims()[2], nkv = kcache.dims()[1], cap = kcache.dims()[2], d = kcache.dims()[3];
    size_t nq = n_heads * d, nk = nkv * d;
    if (kcache.dims()[0] != b || row != nq + 2 * nk || len >= cap)
      bail("attention_step: mismatched shapes " + qkv.shape().str() + " " + kcache.shape().str() + " at position " + std::to_string(len));
    ughip_device* dev = hip_dev(qkv);
    const bool with_rope = cos != nullptr;
    int il = interleaved ? 1 : 0;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 7u : 4u)) bail("attention_step: unexpected number of slices");
      hip_check(ughip_attention_step(dev, hip_raw_slice(*vs[0]), row, 0, nq, nq + nk, hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), hip_raw_slice(*vs.back()), b, n_heads,
                                     nkv, len, cap, d, scale, with_rope ? hip_raw_slice(*vs[3]) : nullptr, with_rope ? hip_raw_slice(*vs[4]) : nullptr,
                                     with_rope ? hip_raw_slice(*vs[5]) : nullptr, il),
                "attention_step");
    };
    std::vector<LB> args = {qkv, kcache, vcache};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return LB::custom(f, args, Shape({b, 1, nq}), qkv.dtype(), qkv.device());
  }

  LB attention_steps(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin, const LB* pos,
                     bool interleaved) const override {
    if (qkv.rank() != 3 || kcache.rank() != 4 || kcache.dims() != vcache.dims()) bail("attention_steps: expected qkv [b, t, row] and caches [b, nkv, cap, d]");
    size_t b = qkv.dims()[0], t = qkv.dims()[1], row = qkv.dims()[2], nkv = kcache.dims()[1], cap = kcache.dims()[2], d = kcache.dims()[3];
    size_t nq = n_heads * d, nk = nkv * d;
    if (kcache.dims()[0] != b || row != nq + 2 * nk)
      bail("attention_steps: mismatched shapes " + qkv.shape().str() + " " + kcache.shape().str());
    if (len + t > cap) bail("attention_steps: " + std::to_string(len + t) + " rows exceed the cache capacity " + std::to_string(cap));
    // one position has a launch of its own kind, and head sizes without a multi-query kernel take the composition
    if (t < 2 || !(d == 32 || d == 64 || d == 128) || qkv.dtype() != DType::F32 || switch_on(SW_NO_APPEND_PAIR))
      return Ops::attention_steps(qkv, kcache, vcache, len, n_heads, scale, cos, sin, pos, interleaved);
    ughip_device* dev = hip_dev(qkv);
    const bool with_rope = cos != nullptr;
    int il = interleaved ? 1 : 0;
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 7u : 4u)) bail("attention_steps: unexpected number of slices");
      ughip_slice *x = hip_raw_slice(*vs[0]), *kc = hip_raw_slice(*vs[1]), *vc = hip_raw_slice(*vs[2]);
      const ughip_slice* c = with_rope ? hip_raw_slice(*vs[3]) : nullptr;
      const ughip_slice* sn = with_rope ? hip_raw_slice(*vs[4]) : nullptr;
      const ughip_slice* p = with_rope ? hip_raw_slice(*vs[5]) : nullptr;
      hip_check(ughip_kv_append_pair(dev, kc, vc, x, nq, nq + nk, row, b, nkv, cap, len, t, d, c, sn, p, il), "attention_steps");
      hip_check(ughip_attention_cached(dev, x, 0, row, kc, vc, hip_raw_slice(*vs.back()), b, n_heads, nkv, t, len + t, cap, d, scale, c, sn, p, il), "attention_steps");
    };
    std::vector<LB> args = {qkv, kcache, vcache};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return LB::custom(f, args, Shape({b, t, nq}), qkv.dtype(), qkv.device());
  }

  LB attention_steps_add(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin, const LB* pos,
                         bool interleaved, const LB& w_o, const LB& residual) const override {
    const bool shapes = qkv.rank() == 3 && kcache.rank() == 4 && kcache.dims() == vcache.dims() && w_o.rank() == 2;
    const size_t b = shapes ? qkv.dims()[0] : 0, t = shapes ? qkv.dims()[1] : 0, row = shapes ? qkv.dims()[2] : 0, nkv = shapes ? kcache.dims()[1] : 0;
    const size_t cap = shapes ? kcache.dims()[2] : 0, d = shapes ? kcache.dims()[3] : 0, nq = n_heads * d, nk = nkv * d, n = shapes ? w_o.dims()[0] : 0, rows = b * t;
    // the shapes the two pieces take on this device, else their composition
    if (!shapes || kcache.dims()[0] != b || row != nq + 2 * nk || len + t > cap || t < 2 || !(d == 32 || d == 64 || d == 128) || qkv.dtype() != DType::F32 ||
        switch_on(SW_NO_APPEND_PAIR) || switch_on(SW_NO_FOLD_EPILOGUES) || (w_o.dtype() != DType::F32 && w_o.dtype() != DType::BF16) || w_o.dims()[1] != nq ||
        rows < (w_o.dtype() == DType::BF16 ? 2u : 9u) || nq % 32 != 0 || n % 8 != 0 || residual.dtype() != DType::F32 || residual.elem_count() != rows * n)
      return Ops::attention_steps_add(qkv, kcache, vcache, len, n_heads, scale, cos, sin, pos, interleaved, w_o, residual);
    ughip_device* dev = hip_dev(qkv);
    const bool with_rope = cos != nullptr;
    const int il = interleaved ? 1 : 0, product = product_for(w_o, nq, rows);
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != (with_rope ? 9u : 6u)) bail("attention_steps_add: unexpected number of slices");
      ughip_slice *x = hip_raw_slice(*vs[0]), *kc = hip_raw_slice(*vs[1]), *vc = hip_raw_slice(*vs[2]);
      const ughip_slice* c = with_rope ? hip_raw_slice(*vs[5]) : nullptr;
      const ughip_slice* sn = with_rope ? hip_raw_slice(*vs[6]) : nullptr;
      const ughip_slice* p = with_rope ? hip_raw_slice(*vs[7]) : nullptr;
      hip_check(ughip_kv_append_pair(dev, kc, vc, x, nq, nq + nk, row, b, nkv, cap, len, t, d, c, sn, p, il), "attention_steps_add");
      hip_check(ughip_attention_cached_linear_add_rows(dev, x, 0, row, kc, vc, b, n_heads, nkv, t, len + t, cap, d, scale, c, sn, p, il, hip_raw_slice(*vs[3]),
                                                       hip_raw_slice(*vs[4]), hip_raw_slice(*vs.back()), n, product),
                "attention_steps_add");
    };
    std::vector<LB> args = {qkv, kcache, vcache, w_o, residual};
    if (with_rope) {
      args.push_back(*cos);
      args.push_back(*sin);
      args.push_back(*pos);
    }
    return LB::custom(f, args, residual.shape(), DType::F32, qkv.device());
  }

  bool device_argmax() const override { return true; }

  LB argmax_into(const LB& token, const LB& logits, size_t row, const LB& ids, const LB& vals, size_t slot) const override {
    if (logits.rank() < 2 || logits.dtype() != DType::F32 || token.dtype() != DType::I32 || token.elem_count() != 1 || ids.dtype() != DType::I32 ||
        vals.dtype() != DType::F32)
      bail("argmax_into: expected F32 logits [.., rows, n], an I32 token, I32 ids and F32 vals");
    size_t n = logits.dims()[logits.rank() - 1];
    if ((row + 1) * n > logits.elem_count() || slot >= ids.elem_count() || 2 * (slot + 1) > vals.elem_count()) bail("argmax_into: row or slot out of range");
    ughip_device* dev = hip_dev(logits);
    // in-place op: arguments first, the token buffer last (schedule.rs:404-413)
    auto f = [=](const std::vector<Slice*>& vs) {
      if (vs.size() != 4) bail("argmax_into: expected 4 slices");
      hip_check(ughip_argmax_row(dev, hip_raw_slice(*vs[0]), n, row, hip_raw_slice(*vs[3]), hip_raw_slice(*vs[1]), hip_raw_slice(*vs[2]), slot), "argmax_into");
    };
    return token.custom_ip(f, {logits, ids, vals});
  }
};

}  // namespace

std::shared_ptr<Ops> hip_ops(bool bf16x3) { return std::make_shared<HipOps>(bf16x3); }

// ---- synthetic weights -----------------------------------------------------------------------------
namespace {
struct SyntheticWeights : WeightSource {
  uint64_t seed;
  float std;
  bool round_bf16;
  float norm_mean, embed_std;  // norm vectors are norm_mean + N(0, std); the embedding table N(0, embed_std) when embed_std > 0
  SyntheticWeights(uint64_t s, float sd, bool r, float nm = 0.f, float es = 0.f) : seed(s), std(sd), round_bf16(r), norm_mean(nm), embed_std(es) {}
  std::vector<float> get(const std::string& name, const std::vector<size_t>& shape) override {
    size_t n = 1;
    for (size_t d : shape) n *= d;
    std::vector<float> out(n);
    uint64_t ts = ugrng::tensor_seed(seed, name);
    const bool is_norm = name.find("norm") != std::string::npos;
    const float mean = is_norm ? norm_mean : 0.f;
    const float std = (embed_std > 0.f && name == "model.embed_tokens.weight") ? embed_std : this->std;
    unsigned nt = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    if (n < (1u << 16)) nt = 1;
    size_t pairs = (n + 1) / 2, per = (pairs + nt - 1) / nt;
    std::vector<std::thread> ths;
    for (unsigned t = 0; t < nt; ++t) {
      size_t p0 = t * per, p1 = std::min(pairs, p0 + per);
      if (p0 >= p1) break;
      ths.emplace_back([&, p0, p1] {
        for (size_t p = p0; p < p1; ++p) {
          double z0, z1;
          ugrng::normal_pair(ts, p, &z0, &z1);
          float a = mean + (float)(z0 * std), b = mean + (float)(z1 * std);
          if (round_bf16) {
            a = bf16_bits_to_f32(f32_to_bf16_bits(a));
            b = bf16_bits_to_f32(f32_to_bf16_bits(b));
          }
          out[2 * p] = a;
          if (2 * p + 1 < n) out[2 * p + 1] = b;
        }
      });
    }
    for (auto& th : ths) th.join();
    return out;
  }
};
}  // namespace

// model.rs:231-244 for one query position, op by op.
LB Ops::attention_decode(const LB& q, const LB& k, const LB& v, float scale) const {
  size_t n_rep = q.dims()[1] / k.dims()[1];
  LB kr = repeat(k, 1, n_rep);
  LB vr = repeat(v, 1, n_rep);
  LB att = q.matmul_t(kr);
  att = att.binary(BinaryOp::Mul, LB::cst(Const::f32(scale), Shape(), q.device()).broadcast(att.shape()));
  return custom_softmax(att).matmul(vr);
}

// model.rs:207-230 for one new position, op by op.
LB Ops::rope_append(const LB& cache, const LB& x, const LB* cos, const LB* sin, const LB* pos, bool interleaved) const {
  size_t n = cache.dims()[1], d = cache.dims()[3];
  LB row = x.split_dim(2, n, d).transpose(2, 1);
  if (cos) row = interleaved ? rope_i(row, *cos, *sin, *pos) : rope(row, *cos, *sin, *pos);
  return cat(cache, row, 2);
}

// model.rs:207-210, 231-245 for one query position, op by op.
LB Ops::attention_decode_flat(const LB& q, const LB& k, const LB& v, float scale, const LB* cos, const LB* sin, const LB* pos, bool interleaved) const {
  size_t d = k.dims()[3], nh = q.dims()[2] / d;
  LB qh = q.split_dim(2, nh, d).transpose(2, 1);
  if (cos) qh = interleaved ? rope_i(qh, *cos, *sin, *pos) : rope(qh, *cos, *sin, *pos);
  return attention_decode(qh, k, v, scale).transpose(2, 1).merge_dims(-2);
}

// model.rs:207-230 for t new positions, op by op (a cache that holds exactly `len` rows).
LB Ops::kv_append(const LB& cache, size_t len, const LB& x, const LB* cos, const LB* sin, const LB* pos, bool interleaved, size_t x_offset,
                  size_t x_row_stride) const {
  if (x_offset != 0 || x_row_stride != 0) bail("kv_append: rows packed into a wider buffer need a device kernel");
  if (cache.rank() != 4 || x.rank() != 3) bail("kv_append: expected cache [b, n, cap, d] and x [b, t, n * d]");
  if (cache.dims()[2] != len) bail("kv_append: this device appends by concatenation and needs a cache of exactly " + std::to_string(len) + " rows, got " + cache.shape().str());
  size_t n = cache.dims()[1], d = cache.dims()[3];
  LB rows = x.split_dim(2, n, d).transpose(2, 1);
  if (cos) rows = interleaved ? rope_i(rows, *cos, *sin, *pos) : rope(rows, *cos, *sin, *pos);
  return cat(cache, rows, 2);
}

// model.rs:207-210, 231-245, op by op.
LB Ops::attention_cached(const LB& q, const LB& k, const LB& v, size_t s, float scale, const LB* cos, const LB* sin, const LB* pos, bool interleaved,
                         size_t q_offset, size_t q_row_stride, size_t n_heads) const {
  if (q_offset != 0 || q_row_stride != 0) bail("attention_cached: rows packed into a wider buffer need a device kernel");
  (void)n_heads;
  if (q.rank() != 3 || k.rank() != 4 || v.rank() != 4) bail("attention_cached: expected q [b, t, nh * d] and k, v [b, nkv, s, d]");
  size_t t = q.dims()[1], d = k.dims()[3], nh = q.dims()[2] / d, nkv = k.dims()[1];
  if (k.dims()[2] != s) bail("attention_cached: this device needs caches of exactly " + std::to_string(s) + " rows, got " + k.shape().str());
  // the reference's causal_mask (cpu_ops.rs:33-56) is only right when the queries are the first t positions
  if (t != 1 && t != s) bail("attention_cached: " + std::to_string(t) + " query positions after " + std::to_string(s - t) + " cached ones need a device kernel");
  LB qh = q.split_dim(2, nh, d).transpose(2, 1);
  if (cos) qh = interleaved ? rope_i(qh, *cos, *sin, *pos) : rope(qh, *cos, *sin, *pos);
  LB kr = repeat(k, 1, nh / nkv);
  LB vr = repeat(v, 1, nh / nkv);
  LB att = qh.matmul_t(kr);
  att = att.binary(BinaryOp::Mul, LB::cst(Const::f32(scale), Shape(), q.device()).broadcast(att.shape()));
  att = t == 1 ? custom_softmax(att) : causal_softmax(att);
  return att.matmul(vr).transpose(2, 1).merge_dims(-2);
}

LB Ops::attention_step(const LB&, const LB&, const LB&, size_t, size_t, float, const LB*, const LB*, const LB*, bool) const {
  bail("attention_step: needs a device with packed projections and caches written in place");
}

LB Ops::attention_steps(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin, const LB* pos,
                        bool interleaved) const {
  if (qkv.rank() != 3 || kcache.rank() != 4 || kcache.dims() != vcache.dims()) bail("attention_steps: expected qkv [b, t, row] and caches [b, nkv, cap, d]");
  const size_t t = qkv.dims()[1], row = qkv.dims()[2], nkv = kcache.dims()[1], d = kcache.dims()[3], nq = n_heads * d, nk = nkv * d;
  if (row != nq + 2 * nk) bail("attention_steps: rows of " + std::to_string(row) + " elements are not q | k | v of " + std::to_string(n_heads) + " and " + std::to_string(nkv) + " heads");
  LB kc = kv_append(kcache, len, qkv, cos, sin, pos, interleaved, nq, row);
  LB vc = kv_append(vcache, len, qkv, nullptr, nullptr, nullptr, false, nq + nk, row);
  return attention_cached(qkv, kc, vc, len + t, scale, cos, sin, pos, interleaved, 0, row, n_heads);
}

LB Ops::argmax_into(const LB&, const LB&, size_t, const LB&, const LB&, size_t) const { bail("argmax_into: this device reads the logits back and picks the token on the host"); }

// A matrix kept in bf16 meets activations of another dtype: matmul wants one dtype throughout
// (ug-core/src/lib.rs:62-70), so the matrix is widened for this use (exact).
LB Ops::linear(const LB& x, const LB& w) const { return x.matmul_t(w.dtype() == x.dtype() ? w : w.cast(x.dtype())); }

// model.rs:206-208 side by side.
LB Ops::linear_packed(const LB& x0, const std::vector<LB>& ws, const LB* alpha, float eps) const {
  if (ws.empty()) bail("linear_packed: no matrices");
  LB x = alpha ? rms_norm(x0, *alpha, eps) : x0;
  LB out = linear(x, ws[0]);
  for (size_t i = 1; i < ws.size(); ++i) out = cat(out, linear(x, ws[i]), x.rank() - 1);
  return out;
}

// model.rs:160-168 up to the down projection.
LB Ops::gate_up(const LB& x0, const LB& w_gate, const LB& w_up, const LB* alpha, float eps) const {
  LB x = alpha ? rms_norm(x0, *alpha, eps) : x0;
  return silu(linear(x, w_gate)).binary(BinaryOp::Mul, linear(x, w_up));
}

// the same from the stacked matrix: SwiGLU on the two halves of the product's rows
LB Ops::gate_up_stacked(const LB& x, const LB& w_gate_up) const {
  const size_t n = w_gate_up.dims()[0] / 2, last = x.rank() - 1;
  LB gu = linear(x, w_gate_up);
  return silu(gu.narrow(last, 0, n)).binary(BinaryOp::Mul, gu.narrow(last, n, n));
}

// model.rs:366-372: a projection, then the residual.
LB Ops::linear_add(const LB& x, const LB& w, const LB& residual) const { return linear(x, w).binary(BinaryOp::Add, residual); }

LB Ops::linear_norm(const LB& x, const LB& alpha, float eps, const LB& w) const { return linear(rms_norm(x, alpha, eps), w); }

LB Ops::attention_steps_add(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin, const LB* pos,
                            bool interleaved, const LB& w_o, const LB& residual) const {
  return linear_add(attention_steps(qkv, kcache, vcache, len, n_heads, scale, cos, sin, pos, interleaved), w_o, residual);
}

LB Ops::mlp_stacked(const LB& x, const LB* alpha, float eps, const LB& w_gate_up, const LB& w_down, const LB& residual) const {
  return linear_add(gate_up_stacked(alpha ? rms_norm(x, *alpha, eps) : x, w_gate_up), w_down, residual);
}

std::shared_ptr<WeightSource> synthetic_weights(uint64_t seed, float std, bool round_bf16, float norm_mean, float embed_std) {
  return std::make_shared<SyntheticWeights>(seed, std, round_bf16, norm_mean, embed_std);
}

LB WeightSource::load(const std::string& name, const std::vector<size_t>& shape, const DevicePtr& dev) {
  std::vector<float> v = get(name, shape);
  size_t n = 1;
  for (size_t d : shape) n *= d;
  if (v.size() != n) bail("unexpected shape for " + name);
  return LB::copy(v.data(), DType::F32, v.size(), Shape(shape), dev);
}

namespace {
struct SafetensorsWeights : WeightSource {
  ug::MmapedSafetensors st;
  explicit SafetensorsWeights(const std::vector<std::string>& paths)
      : st(paths.size() == 1 ? ug::MmapedSafetensors::open(paths[0]) : ug::MmapedSafetensors::multi(paths)) {}
  void check_shape(const std::string& name, const std::vector<size_t>& got, const std::vector<size_t>& want) {
    if (got != want) bail("unexpected shape for " + name + ": " + Shape(got).str() + ", expected " + Shape(want).str());
  }
  std::vector<float> get(const std::string& name, const std::vector<size_t>& shape) override {
    ug::TensorView v = st.get(name);
    check_shape(name, v.shape, shape);
    size_t n = Shape(v.shape).num_elements();
    std::vector<float> out(n);
    DType src = DType::F32;
    if (v.dtype == "BF16") src = DType::BF16;
    else if (v.dtype == "F16") src = DType::F16;
    else if (v.dtype == "I32") src = DType::I32;
    else if (v.dtype == "I64") src = DType::I64;
    else if (v.dtype != "F32") bail("unsupported dtype for " + name + ": " + v.dtype);
    ug::convert_on_host(v.data, src, out.data(), DType::F32, n, name);
    return out;
  }
  LB load(const std::string& name, const std::vector<size_t>& shape, const DevicePtr& dev) override {
    LB lb = st.load_with_cast(name, DType::F32, dev);
    check_shape(name, lb.dims(), shape);
    return lb;
  }
};
}  // namespace

std::shared_ptr<WeightSource> safetensors_weights(const std::vector<std::string>& paths) {
  if (paths.empty()) bail("no safetensors file given");
  return std::make_shared<SafetensorsWeights>(paths);
}

// ---- graph builders (model.rs:32-109) --------------------------------------------------------------------
// model.rs:32-63: hand-written SSA; the ids load is typed F32 although the buffer holds I32,
// so the row offset is (int)((float)id * h).
LB index_select(const LB& src, const LB& ids) {
  DType dtype = DType::F32;
  if (ids.rank() != 2 || src.rank() != 2) bail("index_select: expected rank-2 ids and table");
  size_t b_sz = ids.dims()[0], seq_len = ids.dims()[1], h = src.dims()[1];
  block::Block b;
  uint32_t src_v = b.push(ssa::define_global(0, dtype)).to_varid();
  uint32_t ids_v = b.push(ssa::define_global(1, DType::I32)).to_varid();
  uint32_t dst_v = b.push(ssa::define_global(2, dtype)).to_varid();
  block::Range r1 = b.range(ssa::i32(0), ssa::i32((int32_t)(b_sz * seq_len)), 1);
  block::Id src_off = b.push(ssa::load(ids_v, r1.id().to_a(), dtype));
  src_off = b.mul(src_off, (int32_t)h);
  block::Id dst_off = b.mul(r1.id(), (int32_t)h);
  block::Range r2 = b.range(ssa::i32(0), ssa::i32((int32_t)h), 1);
  block::Id so = b.binary(BinaryOp::Add, src_off.to_a(), r2.id().to_a(), DType::I32);
  block::Id d_o = b.binary(BinaryOp::Add, dst_off.to_a(), r2.id().to_a(), DType::I32);
  block::Id ld = b.push(ssa::load(src_v, so.to_a(), dtype));
  b.push(ssa::store(dst_v, d_o.to_a(), ld.to_a(), dtype));
  b.end_range(r2);
  b.end_range(r1);
  ssa::Kernel k = ssa::Kernel::from_instrs(b.relocate());
  return LB::ssa(k, {src, ids}, Shape({b_sz, seq_len, h}), src.dtype(), src.device());
}

// model.rs:65-78
LB rms_norm(const LB& src, const LB& alpha, float eps) {
  const DevicePtr& dev = src.device();
  size_t rank = src.rank();
  size_t dim_m1 = src.dims()[rank - 1];
  LB sum2 = src.binary(BinaryOp::Mul, src).reduce(ReduceOp::Sum, (long)rank - 1);
  const Shape& s2s = sum2.shape();
  LB m = sum2.binary(BinaryOp::Mul, LB::cst(Const::f32(1.f / (float)dim_m1), s2s, dev))
             .binary(BinaryOp::Add, LB::cst(Const::f32(eps), s2s, dev))
             .unary(UnaryOp::Sqrt);
  return src.binary(BinaryOp::Div, m.broadcast(src.shape())).binary(BinaryOp::Mul, alpha.broadcast(src.shape()));
}

// model.rs:80-92
LB repeat(const LB& lb, size_t axis, size_t n_rep) {
  if (n_rep == 1) return lb;
  if (axis >= lb.rank()) bail("unexpected axis " + std::to_string(axis) + " for repeat " + lb.shape().str());
  LB s = lb.split_dim((long)axis, lb.dims()[axis], 1);
  std::vector<size_t> dims = s.dims();
  dims[axis + 1] = n_rep;
  return s.broadcast(Shape(dims)).merge_dims((long)axis);
}

// model.rs:94-101
LB softmax(const LB& src) {
  const Shape& s = src.shape();
  LB mx = src.reduce(ReduceOp::Max, -1);
  LB diff = src.binary(BinaryOp::Sub, mx.broadcast(s));
  LB e = diff.unary(UnaryOp::Exp);
  LB se = e.reduce(ReduceOp::Sum, -1);
  return e.binary(BinaryOp::Div, se.broadcast(s));
}

// model.rs:103-109
LB silu(const LB& src) {
  LB exp_m = src.unary(UnaryOp::Neg).unary(UnaryOp::Exp);
  LB one = LB::cst(Const::f32(1.f), Shape(), src.device()).broadcast(exp_m.shape());
  LB den = exp_m.binary(BinaryOp::Add, one);
  return src.binary(BinaryOp::Div, den);
}

// model.rs:277-296: theta on the host in f32 powf, then a [max_pos,1]x[1,d/2] matmul, cos/sin.
Rope Rope::create(const Config& cfg, const DevicePtr& dev) {
  size_t head_dim = cfg.head_dim(), max_seq_len = cfg.max_position_embeddings;
  std::vector<float> theta;
  for (size_t i = 0; i < head_dim; i += 2) theta.push_back(1.f / std::pow(cfg.rope_theta, (float)i / (float)head_dim));
  LB theta_lb = LB::copy(theta.data(), DType::F32, theta.size(), Shape({1, head_dim / 2}), dev);
  std::vector<float> idx(max_seq_len);
  for (size_t i = 0; i < max_seq_len; ++i) idx[i] = (float)i;
  LB idx_theta = LB::copy(idx.data(), DType::F32, idx.size(), Shape({max_seq_len, 1}), dev);
  LB mm = idx_theta.matmul(theta_lb);
  return Rope{mm.unary(UnaryOp::Cos), mm.unary(UnaryOp::Sin)};
}

// model.rs:188-197: zero-length caches; with a capacity, buffers of that many rows per head
// (contents undefined until written) that attention appends to in place.
std::vector<Cache> Cache::create(const Config& cfg, const DevicePtr& dev, size_t capacity) {
  std::vector<Cache> c;
  for (size_t i = 0; i < cfg.num_hidden_layers; ++i) {
    Shape s({1, cfg.num_key_value_heads, capacity, cfg.head_dim()});
    Cache one;
    if (capacity) {
      one.prev_k = LB::alloc_uninit(DType::F32, s, dev);
      one.prev_v = LB::alloc_uninit(DType::F32, s, dev);
      one.prev_k.maybe_allocate_uninit();
      one.prev_v.maybe_allocate_uninit();
    } else {
      one.prev_k = LB::cst(Const::f32(0.f), s, dev);
      one.prev_v = LB::cst(Const::f32(0.f), s, dev);
    }
    one.capacity = capacity;
    c.push_back(std::move(one));
  }
  return c;
}

// ---- model (model.rs:299-373) --------------------------------------------------------------------------------
namespace {
LB load_w(WeightSource& w, const std::string& name, const std::vector<size_t>& shape, const DevicePtr& dev) { return w.load(name, shape, dev); }
}  // namespace

Model::Model(const Config& cfg, bool custom_softmax, WeightSource& w, const DevicePtr& dev, std::shared_ptr<Ops> ops)
    : cfg_(cfg), custom_softmax_(custom_softmax), dev_(dev), ops_(std::move(ops)) {
  if (!cfg.tie_word_embeddings) bail("tie_word_embeddings == false is not supported yet");
  size_t h = cfg.hidden_size, isz = cfg.intermediate_size, kv = cfg.head_dim() * cfg.num_key_value_heads;
  embedding_ = load_w(w, "model.embed_tokens.weight", {cfg.vocab_size, h}, dev);
  head_ = embedding_;  // tied (model.rs:315-319)
  ln_f_ = load_w(w, "model.norm.weight", {h}, dev);
  for (size_t i = 0; i < cfg.num_hidden_layers; ++i) {
    std::string p = "model.layers." + std::to_string(i);
    Layer l;
    l.rms1 = load_w(w, p + ".input_layernorm.weight", {h}, dev);
    l.rms2 = load_w(w, p + ".post_attention_layernorm.weight", {h}, dev);
    l.gate_proj = load_w(w, p + ".mlp.gate_proj.weight", {isz, h}, dev);
    l.up_proj = load_w(w, p + ".mlp.up_proj.weight", {isz, h}, dev);
    l.down_proj = load_w(w, p + ".mlp.down_proj.weight", {h, isz}, dev);
    l.q_proj = load_w(w, p + ".self_attn.q_proj.weight", {h, h}, dev);
    l.k_proj = load_w(w, p + ".self_attn.k_proj.weight", {kv, h}, dev);
    l.v_proj = load_w(w, p + ".self_attn.v_proj.weight", {kv, h}, dev);
    l.o_proj = load_w(w, p + ".self_attn.o_proj.weight", {h, h}, dev);
    layers_.push_back(std::move(l));
  }
  rope_ = Rope::create(cfg, dev);
}

// model.rs:203-248
LB Model::attention(const Layer& l, const LB& xs_in, const LB& pos, Cache& cache, const LB* residual, bool norm_first) const {
  if (xs_in.rank() != 3) bail("attention: expected [b, t, hidden]");
  size_t seq_len = xs_in.dims()[1];
  size_t nh = cfg_.num_attention_heads, nkv = cfg_.num_key_value_heads, hd = cfg_.head_dim();
  const float eps = (float)cfg_.rms_norm_eps;
  auto finish = [&](const LB& out) { return residual ? ops_->linear_add(out, l.o_proj, *residual) : ops_->linear(out, l.o_proj); };
  // A preallocated cache is full when its rows are used up: stop here, at graph-build time, like the reference's
  // slice index would (the kernels behind this cannot report an error, and positions past the rotary table
  // would read outside it).
  if (cache.capacity && cache.len + seq_len > cache.capacity)
    bail("attention: " + std::to_string(cache.len) + " cached + " + std::to_string(seq_len) + " new positions exceed the cache's " + std::to_string(cache.capacity) +
         " rows (max_position_embeddings)");
  if (fused_attention_ >= 3 && seq_len == 1 && xs_in.dims()[0] == 1 && cache.capacity && ops_->packed_projections()) {
    // one position: q | k | v come out of one launch (with the norm in front) side by side and are read where they lie
    const size_t nq = nh * hd, nk = nkv * hd, row = nq + 2 * nk, len = cache.len;
    LB qkv = ops_->linear_packed(xs_in, {l.q_proj, l.k_proj, l.v_proj}, norm_first ? &l.rms1 : nullptr, eps);
    cache.len = len + 1;
    const float scale = std::pow((float)hd, -0.5f);
    if (hd >= 16 && hd <= 256 && (hd & (hd - 1)) == 0)
      return finish(ops_->attention_step(qkv, cache.prev_k, cache.prev_v, len, nh, scale, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved));
    LB kc = ops_->kv_append(cache.prev_k, len, qkv, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved, nq, row);
    LB vc = ops_->kv_append(cache.prev_v, len, qkv, nullptr, nullptr, nullptr, false, nq + nk, row);
    return finish(ops_->attention_cached(qkv, kc, vc, cache.len, scale, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved, 0, row, nh));
  }
  if (fused_attention_ >= 3 && cache.capacity && l.qkv_stacked.valid()) {
    // several positions: one product (with the norm in front) gives q | k | v side by side and everything behind it reads
    // its column range of the wide rows in place (a preallocated cache implies a head size the kernels take)
    const size_t len = cache.len;
    LB qkv = norm_first ? ops_->linear_norm(xs_in, l.rms1, eps, l.qkv_stacked) : ops_->linear(xs_in, l.qkv_stacked);
    cache.len = len + seq_len;
    const float scale = std::pow((float)hd, -0.5f);
    if (residual) return ops_->attention_steps_add(qkv, cache.prev_k, cache.prev_v, len, nh, scale, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved, l.o_proj, *residual);
    return finish(ops_->attention_steps(qkv, cache.prev_k, cache.prev_v, len, nh, scale, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved));
  }
  LB xs = norm_first ? rms_norm(xs_in, l.rms1, eps) : xs_in;
  LB q = ops_->linear(xs, l.q_proj);
  LB k = ops_->linear(xs, l.k_proj);
  LB v = ops_->linear(xs, l.v_proj);
  if (fused_attention_ >= 2) {
    // rows go from the projections into the caches (in place when they were preallocated) and
    // the attention kernel reads them there; the result comes back in the layout o_proj reads
    const size_t len = cache.capacity ? cache.len : cache.prev_k.dims()[2];
    LB kc = ops_->kv_append(cache.prev_k, len, k, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved);
    LB vc = ops_->kv_append(cache.prev_v, len, v, nullptr, nullptr, nullptr, false);
    if (cache.capacity == 0) {
      cache.prev_k = kc;
      cache.prev_v = vc;
    }  // else: kc and vc are this step's in-place writes of the storage prev_k / prev_v keep naming
    cache.len = len + seq_len;
    return finish(ops_->attention_cached(q, kc, vc, cache.len, std::pow((float)hd, -0.5f), &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved));
  }
  if (fused_attention_ && seq_len == 1) {
    // one new position: rows go from the projections into the caches and the attention kernel
    // without the split/transpose copies, and the result comes back in the layout o_proj reads
    cache.prev_k = ops_->rope_append(cache.prev_k, k, &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved);
    cache.prev_v = ops_->rope_append(cache.prev_v, v, nullptr, nullptr, nullptr, false);
    return finish(ops_->attention_decode_flat(q, cache.prev_k, cache.prev_v, std::pow((float)hd, -0.5f), &rope_.cos, &rope_.sin, &pos, cfg_.rope_interleaved));
  }
  q = q.split_dim(2, nh, hd).transpose(2, 1);
  k = k.split_dim(2, nkv, hd).transpose(2, 1);
  v = v.split_dim(2, nkv, hd).transpose(2, 1);
  if (cfg_.rope_interleaved) {
    q = ops_->rope_i(q, rope_.cos, rope_.sin, pos);
    k = ops_->rope_i(k, rope_.cos, rope_.sin, pos);
  } else {
    q = ops_->rope(q, rope_.cos, rope_.sin, pos);
    k = ops_->rope(k, rope_.cos, rope_.sin, pos);
  }
  k = ops_->cat(cache.prev_k, k, 2);
  v = ops_->cat(cache.prev_v, v, 2);
  cache.prev_k = k;
  cache.prev_v = v;
  const float scale_v = std::pow((float)hd, -0.5f);
  LB out;
  {
    LB kr = repeat(k, 1, nh / nkv);
    LB vr = repeat(v, 1, nh / nkv);
    LB att = q.matmul_t(kr);
    LB scale = LB::cst(Const::f32(scale_v), Shape(), q.device()).broadcast(att.shape());
    att = att.binary(BinaryOp::Mul, scale);
    if (fused_attention_ && seq_len != 1) {
      att = ops_->causal_softmax(att);
    } else {
      if (seq_len != 1) att = ops_->causal_mask(att);
      att = custom_softmax_ ? ops_->custom_softmax(att) : softmax(att);
    }
    out = att.matmul(vr);
  }
  out = out.transpose(2, 1).merge_dims(-2);
  return finish(out);
}

// model.rs:160-168
LB Model::mlp(const Layer& l, const LB& xs, const LB* residual, bool norm_first) const {
  if (residual && l.gate_up_stacked.valid() && xs.rank() == 3 && xs.dims()[0] * xs.dims()[1] > 1) {
    // several positions: gate and up in one product, SwiGLU on the two halves of its rows, the down projection and the residual
    return ops_->mlp_stacked(xs, norm_first ? &l.rms2 : nullptr, (float)cfg_.rms_norm_eps, l.gate_up_stacked, l.down_proj, *residual);
  }
  if (residual)
    return ops_->linear_add(ops_->gate_up(xs, l.gate_proj, l.up_proj, norm_first ? &l.rms2 : nullptr, (float)cfg_.rms_norm_eps), l.down_proj, *residual);
  LB xs1 = ops_->linear(xs, l.gate_proj);
  LB xs2 = ops_->linear(xs, l.up_proj);
  xs1 = silu(xs1);
  return ops_->linear(xs1.binary(BinaryOp::Mul, xs2), l.down_proj);
}

void Model::set_fused_attention(int level) {
  fused_attention_ = level;
  if (level >= 3 && ops_->packed_projections()) stack_matrices();
}

void Model::stack_matrices() {
  for (Layer& l : layers_) {
    if (l.qkv_stacked.valid() && l.qkv_stacked.dtype() == l.q_proj.dtype()) continue;
    // cat is an allocation written in place (lazy_buffer.rs:722-766), which every schedule would run again:
    // the copy through Id is an ordinary buffer that stays realised
    auto stacked = [](const std::vector<LB>& parts) {
      LB s = LB::cat(parts, 0).unary(UnaryOp::Id);
      s.realize();
      s.detach();
      return s;
    };
    l.qkv_stacked = stacked({l.q_proj, l.k_proj, l.v_proj});
    l.gate_up_stacked = stacked({l.gate_proj, l.up_proj});
  }
}

void Model::store_matrices_bf16() {
  if (bf16_matrices_) return;
  auto narrow = [](LB& w) {
    LB n = w.cast(DType::BF16);
    n.realize();
    n.detach();
    w = n;
  };
  for (Layer& l : layers_)
    for (LB* w : {&l.q_proj, &l.k_proj, &l.v_proj, &l.o_proj, &l.gate_proj, &l.up_proj, &l.down_proj}) narrow(*w);
  narrow(head_);
  if (!layers_.empty() && layers_[0].qkv_stacked.valid()) stack_matrices();  // the stacked copies follow the dtype
  // The lookup reads t rows and keeps an f32 table, the head streams all of the bf16 one; both hold
  // the same values (one tied tensor, model.rs:315-319).
  LB wide = head_.cast(DType::F32);
  wide.realize();
  wide.detach();
  embedding_ = wide;
  bf16_matrices_ = true;
}

std::vector<Cache> Model::new_cache() const {
  return Cache::create(cfg_, dev_, fused_attention_ >= 2 ? ops_->kv_cache_capacity(cfg_.max_position_embeddings, cfg_.head_dim()) : 0);
}

// model.rs:259-269, 365-373
LB Model::fwd(const LB& tokens, const LB& pos, std::vector<Cache>& cache, const std::function<void(const LB&)>* after_layer, bool last_position_only) const {
  if (cache.size() != layers_.size()) bail("cache/layer count mismatch");
  LB xs = index_select(embedding_, tokens);
  float eps = (float)cfg_.rms_norm_eps;
  for (size_t i = 0; i < layers_.size(); ++i) {
    const Layer& l = layers_[i];
    LB residual = xs;
    if (fused_attention_ >= 3) {
      // the norms travel with the projections behind them, the residual adds with the ones in front
      LB h = attention(l, xs, pos, cache[i], &residual, true);
      xs = mlp(l, h, &h, true);
    } else {
      LB h = rms_norm(xs, l.rms1, eps);
      h = attention(l, h, pos, cache[i], nullptr, false);
      h = h.binary(BinaryOp::Add, residual);
      residual = h;
      LB m = rms_norm(h, l.rms2, eps);
      m = mlp(l, m, nullptr, false);
      xs = m.binary(BinaryOp::Add, residual);
    }
    if (after_layer) (*after_layer)(xs);
  }
  if (fused_attention_ >= 3) {
    // a prompt whose logits are read at the last position only: one row through the norm and the head (the row-vector kernel
    // streams the head once, as in a decode step) instead of all of them
    if (last_position_only && xs.rank() == 3 && xs.dims()[1] > 1) xs = xs.narrow(1, xs.dims()[1] - 1, 1);
    return ops_->linear_packed(xs, {head_}, &ln_f_, eps);
  }
  xs = rms_norm(xs, ln_f_, eps);
  return ops_->linear(xs, head_);
}

// One prefill call over the prompt, then `n_steps` greedy single-token steps (graph rebuilt per
// step with a shared CompilationCache, as ug-llama/src/main.rs:124-146 does).  Returns the
// n_steps + 1 argmax ids: one from the prefill logits, one per decode step.
namespace {

// One token step, built and compiled but not yet run.
struct PreparedStep {
  LB tokens, logits;
  size_t t = 0, n_items = 0;
  std::unique_ptr<CompiledSchedule> compiled;
  std::vector<std::unique_ptr<CompiledSchedule>> layers;  // a step launched layer by layer: what ran before `compiled`
  double build_ms = 0, gen_ms = 0, comp_ms = 0;
};

double ms_between(std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) {
  return std::chrono::duration<double, std::milli>(b - a).count();
}

}  // namespace

namespace {

// The same loop for a device that queues work and picks the token itself: the argmax of step i
// writes the input buffer of step i + 1 on the device, so nothing is read back between steps and
// the launches of step i + 1 are issued while step i still runs.  Inputs that have to come from
// the host (prompt, positions) are uploaded before the first launch, because an upload waits for
// the stream.  Ids and the two largest logits of every step are read once at the end.
std::vector<int32_t> generate_greedy_queued(const Model& model, const std::vector<int32_t>& prompt, size_t n_steps, GenerateStats* stats,
                                            const std::vector<int32_t>* forced) {
  using clock = std::chrono::steady_clock;
  const DevicePtr& dev = model.device();
  const Ops& ops = model.ops();
  std::vector<Cache> cache = model.new_cache();
  CompilationCache ccache;
  const bool verbose = switch_on(SW_VERBOSE);
  model.rope().cos.realize();
  model.rope().sin.realize();

  const size_t total = n_steps + 1;
  LB ids = LB::alloc_uninit(DType::I32, Shape({total}), dev), vals = LB::alloc_uninit(DType::F32, Shape({2 * total}), dev);
  ids.maybe_allocate_uninit();
  vals.maybe_allocate_uninit();
  std::vector<LB> tokens(total + 1), pos(total);
  tokens[0] = LB::copy(prompt.data(), DType::I32, prompt.size(), Shape({1, prompt.size()}), dev);
  for (size_t i = 0; i < total; ++i) {
    int32_t p32 = i == 0 ? 0 : (int32_t)(prompt.size() + i - 1);
    pos[i] = LB::copy(&p32, DType::I32, 1, Shape({1, 1}), dev);
    if (forced && i < n_steps) {
      tokens[i + 1] = LB::copy(&(*forced)[i], DType::I32, 1, Shape({1, 1}), dev);  // the input of step i + 1 is given
    } else {
      tokens[i + 1] = LB::alloc_uninit(DType::I32, Shape({1, 1}), dev);  // written by the argmax of step i
      tokens[i + 1].maybe_allocate_uninit();
    }
  }
  LB picked;  // with forced inputs the argmax still runs and is recorded, but writes its id here
  if (forced) {
    picked = LB::alloc_uninit(DType::I32, Shape({1, 1}), dev);
    picked.maybe_allocate_uninit();
  }

  // run_now: every item is launched as soon as it is compiled (the prompt's step: its first kernels execute while the
  // rest of its 300 items are still being looked up)
  const bool by_layer = !switch_on(SW_NO_LAYER_STEPS);
  auto build = [&](size_t i, PreparedStep& st, bool run_now) {
    auto t0 = clock::now();
    st.t = i == 0 ? prompt.size() : 1;
    st.tokens = tokens[i];
    st.n_items = 0;
    // run_now: the hidden state behind every layer is realised as soon as its graph exists, so the device starts on
    // layer 0 after a twentieth of the host work of the step (a prompt of 128 tokens: 0.5 ms of graph and schedule)
    const std::function<void(const LB&)> realise_layer = [&](const LB& x) {
      Schedule part = Schedule::create_one(x);
      st.layers.push_back(std::make_unique<CompiledSchedule>(part.compile_and_run(ccache)));
      st.n_items += part.items().size();
    };
    LB logits = model.fwd(st.tokens, pos[i], cache, run_now && by_layer ? &realise_layer : nullptr, true);
    st.logits = ops.argmax_into(forced ? picked : tokens[i + 1], logits, logits.dims()[logits.rank() - 2] - 1, ids, vals, i);
    auto t1 = clock::now();
    Schedule schedule = Schedule::create_one(st.logits);
    auto t2 = clock::now();
    if (run_now) {
      st.compiled = std::make_unique<CompiledSchedule>(schedule.compile_and_run(ccache));
    } else {
      st.compiled = std::make_unique<CompiledSchedule>(schedule.compile_with_cache(ccache));
      st.compiled->allocate_all();
    }
    st.n_items += schedule.items().size();
    st.build_ms = ms_between(t0, t1);
    st.gen_ms = ms_between(t1, t2);
    st.comp_ms = ms_between(t2, clock::now());
  };

  PreparedStep cur, done;
  auto t_start = clock::now();
  for (Cache& c : cache) {
    c.prev_k.maybe_allocate_uninit();
    c.prev_v.maybe_allocate_uninit();
  }
  build(0, cur, true);
  auto t_decode = t_start;
  for (size_t step = 0; step <= n_steps; ++step) {
    const bool more = step < n_steps;
    PreparedStep next;
    for (Cache& c : cache) {
      c.prev_k.maybe_allocate_uninit();
      c.prev_v.maybe_allocate_uninit();
      c.prev_k.detach();
      c.prev_v.detach();
    }
    auto t0 = clock::now();
    auto t1 = t0;
    if (more) {
      std::exception_ptr run_err;
      std::thread launcher([&] {
        try {
          if (step != 0) cur.compiled->run();  // step 0 was launched while it was compiled
        } catch (...) {
          run_err = std::current_exception();
        }
        t1 = clock::now();
      });
      try {
        build(step + 1, next, false);
        done = PreparedStep();  // buffers go back to the pool; the stream orders their reuse behind this step's kernels
      } catch (...) {
        launcher.join();
        throw;
      }
      launcher.join();
      if (run_err) std::rethrow_exception(run_err);
    } else {
      if (step != 0) cur.compiled->run();
      t1 = clock::now();
    }
    if (verbose)
      fprintf(stderr, "step %zu: own build %.2fms gen %.2fms comp %.2fms; launches %.2fms, next build %.2fms gen %.2fms comp %.2fms, both %.2fms, items %zu (queued, no read-back)\n", step,
              cur.build_ms, cur.gen_ms, cur.comp_ms, ms_between(t0, t1), next.build_ms, next.gen_ms, next.comp_ms, ms_between(t0, clock::now()), cur.n_items);
    if (stats && step != 0) stats->decode_items = cur.n_items;
    if (step == 0) {
      dev->synchronize();  // separates the prompt's time from the decode steps'
      t_decode = clock::now();
      if (stats) stats->prefill_ms = ms_between(t_start, t_decode);
    }
    done = std::move(cur);
    cur = std::move(next);
  }
  std::vector<int32_t> out(total);
  ids.data_vec(out.data(), DType::I32);  // waits for the last step
  if (stats) {
    stats->decode_ms = ms_between(t_decode, clock::now());
    std::vector<float> v(2 * total);
    vals.data_vec(v.data(), DType::F32);
    for (size_t i = 0; i < total; ++i) {
      stats->top1_margin.push_back(v[2 * i] - v[2 * i + 1]);
      stats->top1_value.push_back(v[2 * i]);
    }
    stats->step_ms.assign(n_steps, n_steps ? stats->decode_ms / (double)n_steps : 0.0);  // steps overlap: only their mean is observable
  }
  return out;
}

}  // namespace

// The loop of ug-llama/src/main.rs:118-170 (rebuild the graph, schedule, compile against the cache,
// run, read the logits back, argmax) with one change of order: the graph of step i+1 depends on the
// position but not on the token value, so it is built, scheduled and compiled while the device is
// still executing step i (on a second host thread when the device only queues work, so that it
// also overlaps the launches of step i), and the token id is uploaded into its input buffer once
// known.  Every value computed is the same as in the reference's order.
// UG_LLAMA_NO_OVERLAP=1 keeps everything on the calling thread.
// UG_LLAMA_HOST_ARGMAX=1 keeps this read-back loop on a device that could pick the token itself.
std::vector<int32_t> generate_greedy(const Model& model, const std::vector<int32_t>& prompt, size_t n_steps, GenerateStats* stats,
                                     const std::vector<int32_t>* forced) {
  using clock = std::chrono::steady_clock;
  const Config& cfg = model.config();
  const DevicePtr& dev = model.device();
  if (prompt.empty()) bail("empty prompt");
  if (prompt.size() + n_steps > cfg.max_position_embeddings) bail("prompt + steps exceed max_position_embeddings");
  if (forced && forced->size() != n_steps) bail("forced ids: expected one per decode step (" + std::to_string(n_steps) + "), got " + std::to_string(forced->size()));
  // The embedding gather forms its source offset from the id on the device, where nothing can check it
  // (ids picked by the argmax are in range by construction; these come from the caller).
  auto check_ids = [&](const std::vector<int32_t>& ids, const char* what) {
    for (size_t i = 0; i < ids.size(); ++i)
      if (ids[i] < 0 || (size_t)ids[i] >= cfg.vocab_size)
        bail(std::string(what) + " id " + std::to_string(ids[i]) + " at index " + std::to_string(i) + " is outside the vocabulary of " + std::to_string(cfg.vocab_size));
  };
  check_ids(prompt, "prompt");
  if (forced) check_ids(*forced, "forced");
  if (dev->runs_async() && model.ops().device_argmax() && !switch_on(SW_HOST_ARGMAX) && !switch_on(SW_NO_OVERLAP))
    return generate_greedy_queued(model, prompt, n_steps, stats, forced);
  std::vector<Cache> cache = model.new_cache();
  CompilationCache ccache;
  std::vector<int32_t> out;
  std::vector<float> logits;
  const bool verbose = switch_on(SW_VERBOSE);
  const bool overlap = dev->runs_async() && !switch_on(SW_NO_OVERLAP);
  // The rotary tables are shared by every step: realise them once, before two steps can be in
  // preparation and in flight at the same time.
  model.rope().cos.realize();
  model.rope().sin.realize();

  auto upload_inputs = [&](const std::vector<int32_t>& ids, size_t pos_v, PreparedStep& st, LB& pos) {
    st.t = ids.size();
    st.tokens = LB::copy(ids.data(), DType::I32, st.t, Shape({1, st.t}), dev);
    int32_t p32 = (int32_t)pos_v;
    pos = LB::copy(&p32, DType::I32, 1, Shape({1, 1}), dev);
  };
  auto build = [&](PreparedStep& st, const LB& pos) {
    auto t0 = clock::now();
    st.logits = model.fwd(st.tokens, pos, cache, nullptr, true);  // read at the last position only, like the queued loop
    auto t1 = clock::now();
    Schedule schedule = Schedule::create_one(st.logits);
    auto t2 = clock::now();
    st.compiled = std::make_unique<CompiledSchedule>(schedule.compile_with_cache(ccache));
    // Buffers are taken from the pool here, on the preparing thread, so that the launches of this
    // step (possibly issued from another thread) do not allocate.
    st.compiled->allocate_all();
    st.n_items = schedule.items().size();
    st.build_ms = ms_between(t0, t1);
    st.gen_ms = ms_between(t1, t2);
    st.comp_ms = ms_between(t2, clock::now());
  };

  size_t pos_v = 0;
  PreparedStep cur, done;  // `done`: the previous step, kept until its graph can be freed off the critical path
  auto t_step = clock::now();
  {
    LB pos;
    upload_inputs(prompt, pos_v, cur, pos);
    build(cur, pos);
  }
  for (size_t step = 0; step <= n_steps; ++step) {
    const bool more = step < n_steps;
    PreparedStep next;
    LB next_pos;
    // Host-to-device copies synchronise the stream: the inputs of the next step are uploaded
    // before this step is queued (the token id is a placeholder until the argmax below).
    if (more) upload_inputs({0}, pos_v + cur.t, next, next_pos);
    // The cache buffers this step writes become leaves for the next graph: allocate them now and
    // drop the graph behind them (the compiled schedule keeps what it needs alive), which also
    // keeps the DAG from growing with every step.
    for (Cache& c : cache) {
      c.prev_k.maybe_allocate_uninit();
      c.prev_v.maybe_allocate_uninit();
      c.prev_k.detach();
      c.prev_v.detach();
    }
    // The launches go to a second thread; this thread (whose allocator arena holds the graphs)
    // prepares the next step meanwhile.
    auto t0 = clock::now();
    auto t1 = t0;
    if (more && overlap) {
      std::exception_ptr run_err;
      std::thread launcher([&] {
        try {
          cur.compiled->run();
        } catch (...) {
          run_err = std::current_exception();
        }
        t1 = clock::now();
      });
      try {
        build(next, next_pos);
        done = PreparedStep();
      } catch (...) {
        launcher.join();
        throw;
      }
      launcher.join();
      if (run_err) std::rethrow_exception(run_err);
    } else {
      cur.compiled->run();
      t1 = clock::now();
      if (more) build(next, next_pos);
    }
    auto t2 = clock::now();
    logits.resize(cur.logits.elem_count());
    cur.logits.data_vec(logits.data(), DType::F32);
    auto t3 = clock::now();
    const float* last = logits.data() + (cur.logits.elem_count() / cfg.vocab_size - 1) * cfg.vocab_size;
    size_t best = 0;
    float second = -INFINITY;
    for (size_t i = 1; i < cfg.vocab_size; ++i) {
      if (last[i] > last[best]) {
        second = last[best];
        best = i;
      } else if (last[i] > second) {
        second = last[i];
      }
    }
    if (more) {
      int32_t id = forced ? (*forced)[step] : (int32_t)best;
      next.tokens.data()->slice->copy_host_to_device(&id, DType::I32, 1);
    }
    auto t4 = clock::now();
    if (verbose) {
      // the per-token breakdown ug-llama prints with --verbose (main.rs:154-161)
      fprintf(stderr, "step %zu: run %.2fms, next build %.2fms gen %.2fms comp %.2fms (%s), run+prepare %.2fms, sync+d2h %.2fms, argmax+h2d %.2fms, items %zu\n",
              step, ms_between(t0, t1), next.build_ms, next.gen_ms, next.comp_ms, overlap ? "second thread" : "after the launches", ms_between(t0, t2),
              ms_between(t2, t3), ms_between(t3, t4), cur.n_items);
    }
    double ms = ms_between(t_step, t4);
    t_step = t4;
    if (stats) {
      if (step == 0) stats->prefill_ms = ms;
      else {
        stats->decode_ms += ms;
        stats->step_ms.push_back(ms);
        stats->decode_items = cur.n_items;
      }
      stats->top1_margin.push_back(last[best] - second);
      stats->top1_value.push_back(last[best]);
    }
    pos_v += cur.t;
    out.push_back((int32_t)best);
    done = std::move(cur);
    cur = std::move(next);
  }
  return out;
}

}  // namespace ug_llama
