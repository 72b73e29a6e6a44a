// LazyBuffer builders and realisation.  Mirrors ug-core/src/lazy_buffer.rs: shape rules, error
// conditions and the quirks callers rely on (reduce keeps the input shape, cat on an inner dim
// writes each argument contiguously, in-place ops re-run on every realize).
#include "lazy_buffer.h"

#include <atomic>

namespace ug {

namespace {
size_t fresh_lb_id() {
  static std::atomic<size_t> counter{1};
  return counter.fetch_add(1);
}

LazyBuffer make_lb(Op op, DType dtype, Shape shape, DevicePtr dev, std::shared_ptr<DataCell> data = nullptr) {
  auto inner = std::make_shared<LazyBufferInner>();
  inner->id = fresh_lb_id();
  inner->data = data ? std::move(data) : std::make_shared<DataCell>();
  inner->op = std::move(op);
  inner->dtype = dtype;
  inner->shape = std::move(shape);
  inner->device = std::move(dev);
  return LazyBuffer(std::move(inner));
}
}  // namespace

size_t LazyBuffer::id() const { return p_->id; }
DType LazyBuffer::dtype() const { return p_->dtype; }
const Shape& LazyBuffer::shape() const { return p_->shape; }
const DevicePtr& LazyBuffer::device() const { return p_->device; }
const std::shared_ptr<DataCell>& LazyBuffer::data() const { return p_->data; }

bool LazyBuffer::in_place_op() const { return p_->op.kind == Op::CustomIp || p_->op.kind == Op::Set; }

bool LazyBuffer::realized() const {
  if (in_place_op()) return false;
  return (bool)p_->data->slice;
}

void LazyBuffer::maybe_allocate_uninit() const {
  if (!p_->data->slice) p_->data->slice = p_->device->allocate_uninit(p_->dtype, p_->shape.num_elements());
}

void LazyBuffer::realize() const {
  if (realized()) return;
  Schedule::create_one(*this).compile().run();
}

void LazyBuffer::detach() const {
  if (!realized()) return;
  p_->op = Op();
}

void LazyBuffer::data_vec(void* out, DType dtype) const {
  realize();
  if (!p_->data->slice) bail("no data");
  p_->data->slice->copy_device_to_host(out, dtype, p_->shape.num_elements());
}

std::vector<float> LazyBuffer::data_vec_f32() const {
  std::vector<float> v(elem_count());
  data_vec(v.data(), DType::F32);
  return v;
}

LazyBuffer LazyBuffer::unary(UnaryOp uop) const {
  Op op;
  op.kind = Op::Unary;
  op.unary_op = uop;
  op.arg = *this;
  return make_lb(std::move(op), dtype(), shape(), device());
}

LazyBuffer LazyBuffer::cast(DType dt) const {
  if (dtype() == dt) return *this;
  Op op;
  op.kind = Op::Unary;
  op.unary_op = UnaryOp::Cast;
  op.cast_to = dt;
  op.arg = *this;
  return make_lb(std::move(op), dt, shape(), device());
}

LazyBuffer LazyBuffer::binary(BinaryOp bop, const LazyBuffer& rhs) const {
  if (shape() != rhs.shape()) bail("shape mismatch in binary op, " + shape().str() + " vs " + rhs.shape().str());
  if (dtype() != rhs.dtype()) bail(std::string("dtype mismatch in binary op, ") + dtype_str(dtype()) + " vs " + dtype_str(rhs.dtype()));
  Op op;
  op.kind = Op::Binary;
  op.binary_op = bop;
  op.arg = *this;
  op.arg2 = rhs;
  return make_lb(std::move(op), dtype(), shape(), device());
}

LazyBuffer LazyBuffer::alloc_uninit(DType dtype, const Shape& s, const DevicePtr& dev) {
  Op op;
  op.kind = Op::Value;
  return make_lb(std::move(op), dtype, s, dev);
}

LazyBuffer LazyBuffer::custom(std::function<void(const std::vector<Slice*>&)> f, std::vector<LazyBuffer> args, const Shape& s, DType dtype,
                              const DevicePtr& dev) {
  Op op;
  op.kind = Op::Custom;
  op.f = std::make_shared<std::function<void(const std::vector<Slice*>&)>>(std::move(f));
  op.args = std::move(args);
  return make_lb(std::move(op), dtype, s, dev);
}

LazyBuffer LazyBuffer::custom_ip(std::function<void(const std::vector<Slice*>&)> f, std::vector<LazyBuffer> args) const {
  Op op;
  op.kind = Op::CustomIp;
  op.f = std::make_shared<std::function<void(const std::vector<Slice*>&)>>(std::move(f));
  op.args = std::move(args);
  op.arg2 = *this;
  return make_lb(std::move(op), dtype(), shape(), device(), data());
}

LazyBuffer LazyBuffer::set(const LazyBuffer& values) const {
  if (shape() != values.shape()) bail("shape mismatch in set, " + shape().str() + " vs " + values.shape().str());
  if (dtype() != values.dtype()) bail("dtype mismatch in set");
  Op op;
  op.kind = Op::Set;
  op.arg = values;
  op.arg2 = *this;
  op.dst_layout = Layout::from_shape(shape());
  return make_lb(std::move(op), dtype(), shape(), device(), data());
}

LazyBuffer LazyBuffer::set_l(const LazyBuffer& values, const Layout& dst_layout) const {
  size_t max_offset = dst_layout.offset();
  for (size_t i = 0; i < dst_layout.rank(); ++i) {
    size_t d = dst_layout.dims()[i];
    max_offset += (d ? d - 1 : 0) * dst_layout.strides()[i];
  }
  if (max_offset >= shape().elem_count()) bail("set_l out of bounds, dst shape " + shape().str() + ", max off " + std::to_string(max_offset));
  if (dst_layout.num_elements() != values.shape().elem_count()) bail("set_l mismatch between the values shape " + values.shape().str() + " and layout");
  if (dtype() != values.dtype()) bail("dtype mismatch in set");
  Op op;
  op.kind = Op::Set;
  op.arg = values;
  op.arg2 = *this;
  op.dst_layout = dst_layout;
  return make_lb(std::move(op), dtype(), shape(), device(), data());
}

LazyBuffer LazyBuffer::ssa(const ssa::Kernel& k, std::vector<LazyBuffer> args, const Shape& s, DType dtype, const DevicePtr& dev) {
  Op op;
  op.kind = Op::Ssa;
  op.ssa = k;
  op.args = std::move(args);
  return make_lb(std::move(op), dtype, s, dev);
}

LazyBuffer LazyBuffer::matmul_(const LazyBuffer& rhs, bool transpose) const {
  const auto& ld = dims();
  const auto& rd = rhs.dims();
  size_t dim = ld.size(), rdim = rd.size();
  auto mismatch = [&]() { bail("shape mismatch in matmul " + shape().str() + " " + rhs.shape().str()); };
  if (dim < 2 || rdim < 2) mismatch();
  size_t m = ld[dim - 2], k = ld[dim - 1];
  size_t k2 = transpose ? rd[rdim - 1] : rd[rdim - 2];
  size_t n = transpose ? rd[rdim - 2] : rd[rdim - 1];
  size_t lhs_bsz = 1, rhs_bsz = 1;
  for (size_t i = 0; i + 2 < dim; ++i) lhs_bsz *= ld[i];
  for (size_t i = 0; i + 2 < rdim; ++i) rhs_bsz *= rd[i];
  if (k != k2 || lhs_bsz != rhs_bsz) mismatch();
  std::vector<size_t> out(ld.begin(), ld.end() - 2);
  out.push_back(m);
  out.push_back(n);
  Op op;
  op.kind = Op::MatMul;
  op.arg = *this;
  op.arg2 = rhs;
  op.b = lhs_bsz;
  op.m = m;
  op.n = n;
  op.k = k;
  op.transpose = transpose;
  return make_lb(std::move(op), dtype(), Shape(out), device());
}

// lazy_buffer.rs:453-467: the result keeps the un-reduced shape.
LazyBuffer LazyBuffer::reduce(ReduceOp rop, long dim) const {
  Op op;
  op.kind = Op::Reduce;
  op.reduce_op = rop;
  op.reduce_dim = dim_index(dim, shape(), "reduce");
  op.arg = *this;
  return make_lb(std::move(op), dtype(), shape(), device());
}

LazyBuffer LazyBuffer::split_dim(long dim_, size_t size1, size_t size2) const {
  size_t dim = dim_index(dim_, shape(), "split_dim");
  std::vector<size_t> d = dims();
  size_t size = d[dim];
  d.erase(d.begin() + (long)dim);
  if (size1 * size2 != size) bail("unexpected target sizes for split_dim " + std::to_string(dim));
  d.insert(d.begin() + (long)dim, size2);
  d.insert(d.begin() + (long)dim, size1);
  Op op;
  op.kind = Op::Layout;
  op.layout_op.kind = op::LayoutOp::SplitDim;
  op.layout_op.dim = dim;
  op.layout_op.lhs = dim;
  op.layout_op.rhs = dim + 1;
  op.arg = *this;
  return make_lb(std::move(op), dtype(), Shape(d), device());
}

LazyBuffer LazyBuffer::merge_dims(long dim_) const {
  size_t dim = dim_index(dim_, shape(), "split_dim");
  if (dim + 1 >= rank()) bail("unexpected dim for merge_dims " + std::to_string(dim) + " " + shape().str());
  std::vector<size_t> d = dims();
  size_t size_p = d[dim + 1];
  d.erase(d.begin() + (long)dim + 1);
  d[dim] *= size_p;
  Op op;
  op.kind = Op::Layout;
  op.layout_op.kind = op::LayoutOp::MergeDims;
  op.layout_op.dim = dim;
  op.layout_op.lhs = dim;
  op.layout_op.rhs = dim + 1;
  op.arg = *this;
  return make_lb(std::move(op), dtype(), Shape(d), device());
}

LazyBuffer LazyBuffer::squeeze(long dim_) const {
  size_t dim = dim_index(dim_, shape(), "squeeze");
  std::vector<size_t> d = dims();
  if (d[dim] != 1) bail("cannot squeeze on dim " + std::to_string(dim) + " for shape " + shape().str());
  d.erase(d.begin() + (long)dim);
  return reshape(Shape(d));
}

LazyBuffer LazyBuffer::get_on_dim(long dim_, size_t index) const {
  size_t dim = dim_index(dim_, shape(), "get");
  return narrow((long)dim, index, 1).squeeze((long)dim);
}

LazyBuffer LazyBuffer::unsqueeze(long dim_) const {
  long r = (long)rank();
  long dim = dim_ < 0 ? r + 1 + dim_ : dim_;
  if (dim < 0 || dim > r) bail("unsqueeze: dim out of range");
  std::vector<size_t> d = dims();
  d.insert(d.begin() + dim, 1);
  return reshape(Shape(d));
}

LazyBuffer LazyBuffer::reshape(const Shape& s) const {
  if (s.num_elements() != shape().num_elements())
    bail("cannot reshape between " + shape().str() + " (" + std::to_string(shape().num_elements()) + " elts) and " + s.str() + " (" +
         std::to_string(s.num_elements()) + " elts)");
  Op op;
  op.kind = Op::Reshape;
  op.arg = *this;
  return make_lb(std::move(op), dtype(), s, device());
}

LazyBuffer LazyBuffer::narrow(long dim_, size_t offset, size_t length) const {
  size_t dim = dim_index(dim_, shape(), "narrow");
  size_t size = dims()[dim];
  if (offset + length > size) bail("cannot narrow, offset " + std::to_string(offset) + " + length " + std::to_string(length) + " > size " + std::to_string(size));
  if (offset == 0 && length == size) return *this;
  std::vector<size_t> d = dims();
  d[dim] = length;
  Op op;
  op.kind = Op::Layout;
  op.layout_op.kind = op::LayoutOp::Narrow;
  op.layout_op.dim = dim;
  op.layout_op.offset = offset;
  op.arg = *this;
  return make_lb(std::move(op), dtype(), Shape(d), device());
}

LazyBuffer LazyBuffer::broadcast(const Shape& s) const {
  if (shape().rank() > s.rank()) bail("target shape " + s.str() + " has less dimensions than original shape " + shape().str());
  Op op;
  op.kind = Op::Layout;
  op.layout_op.kind = op::LayoutOp::Broadcast;
  op.layout_op.inserted_dims = s.rank() - shape().rank();
  for (size_t i = 0; i < op.layout_op.inserted_dims; ++i) op.layout_op.broadcasted_dims.push_back(i);
  for (size_t i = 0; i < rank(); ++i) {
    size_t dim_idx = i + op.layout_op.inserted_dims;
    if (s.dims()[dim_idx] != dims()[i]) {
      if (dims()[i] == 1) op.layout_op.broadcasted_dims.push_back(dim_idx);
      else bail("cannot broadcast from " + shape().str() + " to " + s.str());
    }
  }
  op.arg = *this;
  return make_lb(std::move(op), dtype(), s, device());
}

LazyBuffer LazyBuffer::transpose(long d1, long d2) const {
  size_t dim1 = dim_index(d1, shape(), "transpose"), dim2 = dim_index(d2, shape(), "transpose");
  if (dim1 == dim2) return *this;
  std::vector<size_t> d = dims();
  std::swap(d[dim1], d[dim2]);
  Op op;
  op.kind = Op::Layout;
  op.layout_op.kind = op::LayoutOp::Transpose;
  op.layout_op.dim1 = dim1;
  op.layout_op.dim2 = dim2;
  op.arg = *this;
  return make_lb(std::move(op), dtype(), Shape(d), device());
}

LazyBuffer LazyBuffer::cst(const Const& c, const Shape& s, const DevicePtr& dev) {
  Op op;
  op.kind = Op::Const;
  op.cst = c;
  return make_lb(std::move(op), c.dtype, s, dev);
}

LazyBuffer LazyBuffer::from_slice(std::unique_ptr<Slice> data, const Shape& s, const DevicePtr& dev) {
  if (s.num_elements() != data->len()) bail("unexpected number of elements " + std::to_string(data->len()) + " for shape " + s.str());
  DType dt = data->dtype();
  auto cell = std::make_shared<DataCell>();
  cell->slice = std::move(data);
  Op op;
  op.kind = Op::Value;
  return make_lb(std::move(op), dt, s, dev, cell);
}

LazyBuffer LazyBuffer::copy(const void* data, DType dtype, size_t len, const Shape& s, const DevicePtr& dev) {
  if (s.num_elements() != len) bail("unexpected number of elements " + std::to_string(len) + " for shape " + s.str());
  std::unique_ptr<Slice> slice = dev->allocate_uninit(dtype, len);
  slice->copy_host_to_device(data, dtype, len);
  return from_slice(std::move(slice), s, dev);
}

// lazy_buffer.rs:722-766
LazyBuffer LazyBuffer::cat(const std::vector<LazyBuffer>& args, long dim_) {
  if (args.empty()) bail("empty list in cat");
  const LazyBuffer& arg0 = args[0];
  if (args.size() == 1) return arg0;
  size_t dim = dim_index(dim_, arg0.shape(), "cat");
  std::vector<size_t> dims = arg0.dims();
  dims[dim] = 0;
  for (const LazyBuffer& arg : args) {
    if (arg.dtype() != arg0.dtype()) bail("mismatch between dtypes in cat");
    if (arg.rank() != arg0.rank()) bail("mismatch between ranks in cat");
    dims[dim] += arg.dims()[dim];
    for (size_t i = 0; i < dims.size(); ++i)
      if (i != dim && dims[i] != arg.dims()[i]) bail("mismatch between shapes in cat on dim " + std::to_string(dim) + ", arg0: " + arg0.shape().str() + ", arg: " + arg.shape().str());
  }
  size_t stride = 1;
  for (size_t i = dim + 1; i < dims.size(); ++i) stride *= dims[i];
  size_t offset = 0;
  LazyBuffer vs = alloc_uninit(arg0.dtype(), Shape(dims), arg0.device());
  for (const LazyBuffer& arg : args) {
    Layout l = Layout::from_shape(arg.shape());
    l.set_offset(offset * stride);
    vs = vs.set_l(arg, l);
    offset += arg.dims()[dim];
  }
  return vs;
}

}  // namespace ug
