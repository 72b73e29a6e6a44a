// The accelerator boundary: `trait Slice` and `trait Device` of ug-core/src/lib.rs:29-73 as
// abstract classes.  Backends: HipDevice (hip_device.cpp, over the C ABI of include/ughip.h).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "lang.h"

namespace ug {

struct Device;

// lib.rs:29-47
struct Slice {
  virtual ~Slice() = default;
  virtual DType dtype() const = 0;
  virtual size_t len() const = 0;
  // Errors on dtype or length mismatch; the data is in place when the call returns.
  virtual void copy_host_to_device(const void* src, DType dtype, size_t len) = 0;
  virtual void copy_device_to_host(void* dst, DType dtype, size_t len) const = 0;
  bool is_empty() const { return len() == 0; }
};

// Device::Func
struct Func {
  virtual ~Func() = default;
};

// lib.rs:49-73
struct Device {
  virtual ~Device() = default;
  virtual std::unique_ptr<Slice> allocate_uninit(DType dtype, size_t len) = 0;
  virtual void synchronize() = 0;
  virtual std::shared_ptr<Func> compile(const ssa::Kernel& kernel, const std::string* name) = 0;
  virtual void run(Func& f, const std::vector<Slice*>& args) = 0;
  virtual void matmul(Slice& dst, const Slice& lhs, const Slice& rhs, size_t b, size_t m, size_t n, size_t k, const Layout& lhs_l,
                      const Layout& rhs_l) = 0;
  virtual bool use_grid() const = 0;
  virtual const char* name() const = 0;
  // True when run/matmul only queue work (results are ready after synchronize or a copy back).
  virtual bool runs_async() const { return false; }
  // Element type conversion between two slices of equal length, if the device can do it in its
  // own memory; false = not offered (the caller converts on the host).
  virtual bool convert(Slice& dst, const Slice& src) {
    (void)dst;
    (void)src;
    return false;
  }
};

}  // namespace ug
