// LazyBuffer DAG and scheduler.  Mirrors ug-core/src/{lazy_buffer,schedule,cache}.rs.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "device.h"
#include "lang.h"

namespace ug {

using DevicePtr = std::shared_ptr<Device>;
// lazy_buffer.rs:5: Fn(Vec<&mut Slice>) -> Result<()>
using CustomF = std::shared_ptr<std::function<void(const std::vector<Slice*>&)>>;

struct LazyBufferInner;

// The storage cell an `Arc<RefCell<Option<D::Slice>>>` stands for; shared by in-place ops.
struct DataCell {
  std::unique_ptr<Slice> slice;
};

// lazy_buffer.rs:85-112
class LazyBuffer {
 public:
  LazyBuffer() = default;
  explicit LazyBuffer(std::shared_ptr<LazyBufferInner> p) : p_(std::move(p)) {}
  bool valid() const { return (bool)p_; }
  const LazyBufferInner& inner() const { return *p_; }

  size_t id() const;
  DType dtype() const;
  const Shape& shape() const;
  const std::vector<size_t>& dims() const { return shape().dims(); }
  size_t rank() const { return shape().rank(); }
  size_t elem_count() const { return shape().num_elements(); }
  const DevicePtr& device() const;
  const std::shared_ptr<DataCell>& data() const;

  bool in_place_op() const;                // lazy_buffer.rs:130-144
  bool realized() const;                   // :146-154
  void maybe_allocate_uninit() const;      // :116-124
  void realize() const;                    // :156-164
  // Once realised a buffer is a leaf for every later schedule (:146-154); forget how it was made
  // so the graph behind it can be freed.  No-op for unrealised or in-place buffers.
  void detach() const;
  // :170-183 -- realize, then copy to `out` (elem_count() elements of `dtype`).
  void data_vec(void* out, DType dtype) const;
  std::vector<float> data_vec_f32() const;

  // builders (lazy_buffer.rs:229-766)
  LazyBuffer unary(UnaryOp op) const;
  LazyBuffer cast(DType dtype) const;
  LazyBuffer binary(BinaryOp op, const LazyBuffer& rhs) const;
  static LazyBuffer alloc_uninit(DType dtype, const Shape& s, const DevicePtr& dev);
  static LazyBuffer custom(std::function<void(const std::vector<Slice*>&)> f, std::vector<LazyBuffer> args, const Shape& s, DType dtype,
                           const DevicePtr& dev);
  LazyBuffer custom_ip(std::function<void(const std::vector<Slice*>&)> f, std::vector<LazyBuffer> args) const;
  LazyBuffer set(const LazyBuffer& values) const;
  LazyBuffer set_l(const LazyBuffer& values, const Layout& dst_layout) const;
  static LazyBuffer ssa(const ssa::Kernel& k, std::vector<LazyBuffer> args, const Shape& s, DType dtype, const DevicePtr& dev);
  LazyBuffer matmul(const LazyBuffer& rhs) const { return matmul_(rhs, false); }
  LazyBuffer matmul_t(const LazyBuffer& rhs) const { return matmul_(rhs, true); }
  LazyBuffer matmul_(const LazyBuffer& rhs, bool transpose) const;
  LazyBuffer reduce(ReduceOp op, long dim) const;
  LazyBuffer split_dim(long dim, size_t size1, size_t size2) const;
  LazyBuffer merge_dims(long dim) const;
  LazyBuffer squeeze(long dim) const;
  LazyBuffer get_on_dim(long dim, size_t index) const;
  LazyBuffer get(size_t index) const { return get_on_dim(0, index); }
  LazyBuffer unsqueeze(long dim) const;
  LazyBuffer reshape(const Shape& s) const;
  LazyBuffer narrow(long dim, size_t offset, size_t length) const;
  LazyBuffer broadcast(const Shape& s) const;
  LazyBuffer transpose(long dim1, long dim2) const;
  static LazyBuffer cst(const Const& c, const Shape& s, const DevicePtr& dev);
  static LazyBuffer from_slice(std::unique_ptr<Slice> data, const Shape& s, const DevicePtr& dev);
  static LazyBuffer copy(const void* data, DType dtype, size_t len, const Shape& s, const DevicePtr& dev);
  static LazyBuffer cat(const std::vector<LazyBuffer>& args, long dim);

 private:
  std::shared_ptr<LazyBufferInner> p_;
};

// lazy_buffer.rs:50-83
struct Op {
  enum Kind { Unary, Binary, MatMul, Reduce, Const, Value, Layout, Reshape, Custom, CustomIp, Ssa, Set } kind = Value;
  UnaryOp unary_op = UnaryOp::Id;
  DType cast_to = DType::F32;
  BinaryOp binary_op = BinaryOp::Add;
  ReduceOp reduce_op = ReduceOp::Sum;
  size_t reduce_dim = 0;
  ug::Const cst;
  op::LayoutOp layout_op;
  size_t b = 0, m = 0, n = 0, k = 0;  // MatMul
  bool transpose = false;
  CustomF f;
  ssa::Kernel ssa;
  ug::Layout dst_layout;          // Set
  LazyBuffer arg, arg2;           // Unary/Layout/Reshape/Reduce: arg; Binary/MatMul: (arg, arg2); Set: values = arg, src = arg2; CustomIp: src = arg2
  std::vector<LazyBuffer> args;   // Custom / CustomIp / Ssa
};

struct LazyBufferInner {
  size_t id = 0;
  std::shared_ptr<DataCell> data;
  Op op;
  DType dtype = DType::F32;
  Shape shape;
  DevicePtr device;
};

// ---- schedule.rs ---------------------------------------------------------------------------
using Args = std::vector<std::pair<ArgId, LazyBuffer>>;

// schedule.rs:7-40
struct KernelItem {
  op::Ast ast;
  std::pair<ArgId, LazyBuffer> dst;
  bool has_dst_layout = false;
  Layout dst_layout;
  Args args;
  op::Kernel kernel() const;
};

// schedule.rs:42-59
struct ScheduleItem {
  enum Kind { Kernel, MatMul, Custom, Ssa } kind = Kernel;
  KernelItem kernel;
  LazyBuffer dst, lhs, rhs;
  size_t b = 0, m = 0, n = 0, k = 0;
  bool transpose = false;
  CustomF f;
  ssa::Kernel ssa;
  Args args;
};

// cache.rs:74-101
struct CompilationCache {
  std::unordered_map<std::string, std::shared_ptr<Func>> op_cache, ssa_cache;
};

// schedule.rs:210-306
struct CompiledFunc {
  enum Kind { Kernel, MatMul, Custom } kind = Kernel;
  std::shared_ptr<Func> func;
  Args args;
  LazyBuffer dst, lhs, rhs;
  size_t b = 0, m = 0, n = 0, k = 0;
  bool transpose = false;
  CustomF f;
};

struct CompiledSchedule {
  std::vector<CompiledFunc> funcs;
  DevicePtr device;
  void run() const;
  void run_one(const CompiledFunc& f) const;
  // Allocates every buffer run() would allocate lazily (schedule.rs:247-250, 268-270), so that a
  // later run() only dispatches.
  void allocate_all() const;
};

// schedule.rs:61-208
class Schedule {
 public:
  static Schedule create(const std::vector<LazyBuffer>& buffers);
  static Schedule create_one(const LazyBuffer& b) { return create({b}); }
  const std::vector<ScheduleItem>& items() const { return items_; }
  CompiledSchedule compile() const {
    CompilationCache c;
    return compile_with_cache(c);
  }
  CompiledSchedule compile_with_cache(CompilationCache& cache) const;
  // The same, and every item is dispatched as soon as it is compiled: on a device that queues work the first kernels
  // execute while the later items are still being looked up.  The result is as after compile_with_cache + run().
  CompiledSchedule compile_and_run(CompilationCache& cache) const;
  const LazyBuffer& get_arg_id(ArgId id) const;

 private:
  CompiledFunc compile_item(const ScheduleItem& item, CompilationCache& cache) const;
  std::vector<ScheduleItem> items_;
  std::map<size_t, LazyBuffer> per_arg_id_;
  DevicePtr device_;
};

// Key of the op cache: the kernel with argument ids renumbered 0..n (cache.rs:14-72).
std::string normalized_kernel_key(const op::Kernel& k);

}  // namespace ug
