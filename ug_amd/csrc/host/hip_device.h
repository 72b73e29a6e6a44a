#pragma once
#include "ug/device.h"
#include "ughip.h"

namespace ug {

class HipSlice : public Slice {
 public:
  explicit HipSlice(ughip_slice* s) : s_(s) {}
  ~HipSlice() override;
  DType dtype() const override;
  size_t len() const override;
  void copy_host_to_device(const void* src, DType dtype, size_t len) override;
  void copy_device_to_host(void* dst, DType dtype, size_t len) const override;
  ughip_slice* raw() const { return s_; }

 private:
  ughip_slice* s_;
};

class HipFunc : public Func {
 public:
  explicit HipFunc(ughip_func* f) : f_(f) {}
  ~HipFunc() override;
  ughip_func* raw() const { return f_; }

 private:
  ughip_func* f_;
};

class HipDevice : public Device {
 public:
  explicit HipDevice(int ordinal);
  ~HipDevice() override;
  std::unique_ptr<Slice> allocate_uninit(DType dtype, size_t len) override;
  void synchronize() override;
  std::shared_ptr<Func> compile(const ssa::Kernel& kernel, const std::string* name) override;
  void run(Func& f, const std::vector<Slice*>& args) override;
  void matmul(Slice& dst, const Slice& lhs, const Slice& rhs, size_t b, size_t m, size_t n, size_t k, const Layout& lhs_l,
              const Layout& rhs_l) override;
  // The backend re-parallelises serial loop nests itself (ug-core/src/schedule.rs:162).
  bool use_grid() const override { return false; }
  bool runs_async() const override { return true; }
  bool convert(Slice& dst, const Slice& src) override;
  const char* name() const override { return "hip"; }
  ughip_device* raw() const { return d_; }

 private:
  ughip_device* d_ = nullptr;
};

ughip_slice* hip_raw_slice(const Slice& s);

}  // namespace ug
