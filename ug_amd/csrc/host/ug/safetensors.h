// Memory-mapped safetensors files -> device buffers: ug-core/src/safetensors.rs as C++.
//
// File format (safetensors 0.4, the crate ug-core depends on): 8-byte little-endian header length
// N, N bytes of JSON {"name": {"dtype": "F32", "shape": [..], "data_offsets": [begin, end]}, ...,
// "__metadata__": {..}}, then the data; offsets are relative to the end of the header.
//
// load_with_cast differs from the reference in where the conversion runs: when the device offers
// Device::convert (the HIP device does), the tensor is uploaded in its stored dtype and converted
// in device memory; otherwise it is converted on the host first, as safetensors.rs:141-271 does.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "lazy_buffer.h"

namespace ug {

struct TensorView {
  std::string dtype;  // as spelled in the file: "F32", "BF16", "U8", ...
  std::vector<size_t> shape;
  const uint8_t* data = nullptr;
  size_t nbytes = 0;
};

class MmapedSafetensors {
 public:
  // safetensors.rs:21-35
  static MmapedSafetensors open(const std::string& path);
  // safetensors.rs:44-69: a name that appears in several files resolves to the last one.
  static MmapedSafetensors multi(const std::vector<std::string>& paths);

  LazyBuffer load(const std::string& name, const DevicePtr& dev) const;                             // :71-74
  LazyBuffer load_with_cast(const std::string& name, DType dtype, const DevicePtr& dev) const;      // :76-84
  std::pair<Shape, std::unique_ptr<Slice>> load_slice(const std::string& name, const DevicePtr& dev) const;  // :86-121
  std::pair<Shape, std::unique_ptr<Slice>> load_slice_with_cast(const std::string& name, DType dtype, const DevicePtr& dev) const;  // :123-273
  std::vector<std::pair<std::string, TensorView>> tensors() const;  // :275-281
  TensorView get(const std::string& name) const;                    // :283-295

  // Where the last load_with_cast converted: true = on the device.
  bool last_cast_on_device() const { return last_cast_on_device_; }

 private:
  struct File;
  static std::shared_ptr<File> open_file(const std::string& path);
  std::vector<std::shared_ptr<File>> files_;
  bool routed_ = false;
  std::map<std::string, size_t> routing_;
  mutable bool last_cast_on_device_ = false;
};

// The element conversions of safetensors.rs:141-271 on the host: `n` elements of `src_dtype` at
// `src` (any alignment) into `dst` (`dst_dtype`).
void convert_on_host(const uint8_t* src, DType src_dtype, void* dst, DType dst_dtype, size_t n, const std::string& name);

}  // namespace ug
