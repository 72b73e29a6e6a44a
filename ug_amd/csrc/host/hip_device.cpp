// HipDevice: ug::Device / ug::Slice over the C ABI of include/ughip.h -- what the Rust `ug-hip`
// crate does with `extern "C"`, written in C++.  Counterpart of ug-cuda/src/runtime.rs:212-393.
#include "hip_device.h"

namespace ug {

namespace {
[[noreturn]] void fail(const char* what) { bail(std::string(what) + ": " + ughip_last_error()); }
}  // namespace

HipSlice::~HipSlice() { ughip_free(s_); }
DType HipSlice::dtype() const { return (DType)ughip_slice_dtype(s_); }
size_t HipSlice::len() const { return ughip_slice_len(s_); }
void HipSlice::copy_host_to_device(const void* src, DType dtype, size_t len) {
  if (ughip_h2d(s_, src, (int)dtype, len)) fail("copy_host_to_device");
}
void HipSlice::copy_device_to_host(void* dst, DType dtype, size_t len) const {
  if (ughip_d2h(s_, dst, (int)dtype, len)) fail("copy_device_to_host");
}

HipFunc::~HipFunc() { ughip_func_release(f_); }

HipDevice::HipDevice(int ordinal) {
  if (ughip_device_create(ordinal, &d_)) fail("HipDevice::new");
}
HipDevice::~HipDevice() { ughip_device_release(d_); }

std::unique_ptr<Slice> HipDevice::allocate_uninit(DType dtype, size_t len) {
  ughip_slice* s = nullptr;
  if (ughip_alloc(d_, (int)dtype, len, &s)) fail("allocate_uninit");
  return std::unique_ptr<Slice>(new HipSlice(s));
}

void HipDevice::synchronize() {
  if (ughip_synchronize(d_)) fail("synchronize");
}

std::shared_ptr<Func> HipDevice::compile(const ssa::Kernel& kernel, const std::string* name) {
  ughip_ssa wire = kernel.wire();
  ughip_func* f = nullptr;
  if (ughip_compile(d_, &wire, name ? name->c_str() : nullptr, &f)) fail("compile");
  return std::make_shared<HipFunc>(f);
}

static ughip_slice* raw_slice(const Slice& s) {
  const HipSlice* h = dynamic_cast<const HipSlice*>(&s);
  if (!h) bail("slice does not belong to the hip device");
  return h->raw();
}

void HipDevice::run(Func& f, const std::vector<Slice*>& args) {
  HipFunc* hf = dynamic_cast<HipFunc*>(&f);
  if (!hf) bail("func does not belong to the hip device");
  std::vector<ughip_slice*> raws;
  raws.reserve(args.size());
  for (Slice* s : args) raws.push_back(raw_slice(*s));
  if (ughip_run(d_, hf->raw(), raws.data(), raws.size())) fail("run");
}

void HipDevice::matmul(Slice& dst, const Slice& lhs, const Slice& rhs, size_t b, size_t m, size_t n, size_t k, const Layout& lhs_l,
                       const Layout& rhs_l) {
  if (lhs_l.rank() != rhs_l.rank()) bail("matmul: layouts of different rank");
  if (ughip_matmul(d_, raw_slice(dst), raw_slice(lhs), raw_slice(rhs), b, m, n, k, lhs_l.rank(), lhs_l.dims().data(), lhs_l.strides().data(), lhs_l.offset(),
                   rhs_l.dims().data(), rhs_l.strides().data(), rhs_l.offset()))
    fail("matmul");
}

bool HipDevice::convert(Slice& dst, const Slice& src) {
  if (ughip_convert(d_, raw_slice(src), raw_slice(dst))) fail("convert");
  return true;
}

ughip_slice* hip_raw_slice(const Slice& s) { return raw_slice(s); }

}  // namespace ug
