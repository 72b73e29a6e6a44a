// ORACLE -- TEST INFRASTRUCTURE ONLY (see cpu_device.cpp).  Declarations shared by the oracle's
// translation units.  Uses the front-end's abstract ug::Device so the same graphs run on both.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "llama.h"
#include "ug/device.h"
#include "ug/lazy_buffer.h"

namespace ug_oracle {

// ug::CpuStorage (ug-core/src/cpu_runtime.rs:6-12): a typed host vector.
class CpuSlice : public ug::Slice {
 public:
  CpuSlice(ug::DType dt, size_t len);
  ug::DType dtype() const override { return dtype_; }
  size_t len() const override { return len_; }
  void copy_host_to_device(const void* src, ug::DType dtype, size_t len) override;
  void copy_device_to_host(void* dst, ug::DType dtype, size_t len) const override;
  char* data() { return bytes_.data(); }
  const char* data() const { return bytes_.data(); }

 private:
  ug::DType dtype_;
  size_t len_;
  std::vector<char> bytes_;
};

CpuSlice& cpu_slice(ug::Slice& s);
const CpuSlice& cpu_slice(const ug::Slice& s);

// ug::CpuDevice (cpu_runtime.rs:248-359)
class CpuDevice : public ug::Device {
 public:
  std::unique_ptr<ug::Slice> allocate_uninit(ug::DType dtype, size_t len) override;
  void synchronize() override {}
  std::shared_ptr<ug::Func> compile(const ug::ssa::Kernel& kernel, const std::string* name) override;
  void run(ug::Func& f, const std::vector<ug::Slice*>& args) override;
  void matmul(ug::Slice& dst, const ug::Slice& lhs, const ug::Slice& rhs, size_t b, size_t m, size_t n, size_t k, const ug::Layout& lhs_l,
              const ug::Layout& rhs_l) override;
  bool use_grid() const override { return false; }
  const char* name() const override { return "cpu"; }
  std::shared_ptr<ug::Func> compile_c(const std::string& c_code, const std::string& func_name);
};

std::string gen_c(const std::string& func_name, const ug::ssa::Kernel& kernel);
std::string func_c_code(const ug::Func& f);

// ug-llama/src/cpu_ops.rs
std::shared_ptr<ug_llama::Ops> cpu_ops();

// ug-core/src/interpreter.rs: one block of `n_lanes` threads, `grid_idx` = blockIdx.
struct InterpBuffer {
  ug::DType dtype;
  void* data;
  size_t len;
};
void eval_ssa(const ug::ssa::Kernel& kernel, std::vector<InterpBuffer>& buffers, size_t n_lanes, size_t grid_idx);

}  // namespace ug_oracle
