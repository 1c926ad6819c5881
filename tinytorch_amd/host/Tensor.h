// Minimal value-semantic Tensor for the attention path: the part of TinyTorch's tensor core that
// function::sdpAttention touches (reference src/Tensor/Tensor.h:26-284, TensorImpl.h:19-98, Storage.cpp:19-79,
// Options.h:36-85, DType.h:20-28, Device.h:13-49).  Tensors are dense row-major; a Tensor is a shared handle to
// its implementation; device memory comes from a size-bucketed caching allocator (512-byte rounding, as
// reference src/Tensor/CachedAllocator.cpp:24-28) on top of hipMalloc.
#pragma once

#include <cstdint>
#include <cstring>
#include <memory>
#include <optional>
#include <string>
#include <vector>

#include "Macros.h"

namespace tinytorch {

// Numbering is the dispatch-table layout of the reference (src/Tensor/DType.h:20-28).
enum class DType : uint8_t { Float32 = 0, Float16 = 1, BFloat16 = 2, Int32 = 3, Int64 = 4, Bool = 5, DTypeCount };
// Slot 1 is the accelerator slot (the reference calls it CUDA, src/Tensor/Device.h:13-17); here it holds the HIP
// implementation and nothing else.
enum class DeviceType : uint8_t { CPU = 0, GPU = 1, CUDA = GPU, DeviceTypeCount = 2 };
using DeviceIndex = int8_t;

size_t dtypeSize(DType t);
const char* dtypeToString(DType t);
const char* deviceTypeToString(DeviceType t);

struct Device {
  DeviceType type = DeviceType::CPU;
  DeviceIndex index = 0;
  Device() = default;
  Device(DeviceType t, DeviceIndex i = 0) : type(t), index(i) {}
  bool isCpu() const { return type == DeviceType::CPU; }
  bool isGpu() const { return type == DeviceType::GPU; }
  bool operator==(const Device& o) const { return type == o.type && index == o.index; }
  bool operator!=(const Device& o) const { return !(*this == o); }
};

void setDefaultDevice(Device d);
Device getDefaultDevice();

struct Options {
  Device device_;
  DType dtype_ = DType::Float32;
  bool requiresGrad_ = false;
  Options() : device_(getDefaultDevice()) {}
  Options& device(Device d) { device_ = d; return *this; }
  Options& dtype(DType t) { dtype_ = t; return *this; }
  Options& requiresGrad(bool r = true) { requiresGrad_ = r; return *this; }
  Options noGrad() const { Options o = *this; o.requiresGrad_ = false; return o; }
};
namespace options {
inline Options device(DeviceType t, DeviceIndex i = 0) { return Options().device(Device(t, i)); }
inline Options dtype(DType t) { return Options().dtype(t); }
}  // namespace options

// Owning byte buffer on one device.
class Storage {
 public:
  Storage(size_t nbytes, Device device);
  ~Storage();
  Storage(const Storage&) = delete;
  Storage& operator=(const Storage&) = delete;
  void* data() const { return data_; }
  size_t nbytes() const { return nbytes_; }
  Device device() const { return device_; }
  static void copy(void* dst, Device dstDev, const void* src, Device srcDev, size_t nbytes);

 private:
  void* data_ = nullptr;
  size_t nbytes_ = 0;
  Device device_;
};

// Bytes currently cached (free) / handed out by the device allocator of `device`; for tests and diagnostics.
size_t deviceAllocatorCachedBytes(DeviceIndex device);
size_t deviceAllocatorLiveBytes(DeviceIndex device);
void deviceAllocatorRelease(DeviceIndex device);

struct FunctionBase;  // autograd node (Function.h)

class Tensor {
 public:
  Tensor() = default;
  Tensor(const std::vector<int64_t>& shape, Options options);
  template <typename T>
  explicit Tensor(const std::vector<T>& values) : Tensor(values, {static_cast<int64_t>(values.size())}, Options()) {}
  template <typename T>
  Tensor(const std::vector<T>& values, const std::vector<int64_t>& shape, Options options = Options());

  static Tensor empty(const std::vector<int64_t>& shape, Options options = Options()) { return Tensor(shape, options); }
  static Tensor zeros(const std::vector<int64_t>& shape, Options options = Options());
  static Tensor ones(const std::vector<int64_t>& shape, Options options = Options());
  static Tensor scalar(float value, Options options = Options());

  bool defined() const { return impl_ != nullptr; }
  const std::vector<int64_t>& shape() const;
  int64_t dim() const { return static_cast<int64_t>(shape().size()); }
  int64_t size(int64_t d) const;  // negative d counts from the back
  int64_t numel() const;
  DType dtype() const;
  Device device() const;
  Options options() const;
  bool requiresGrad() const;
  void setRequiresGrad(bool r);
  std::shared_ptr<FunctionBase> gradFn() const;
  void setGradFn(std::shared_ptr<FunctionBase> fn);
  // Gradient slot of a tensor that requires grad (reference src/Tensor/Tensor.h grad()/addGrad()).  This layer has no
  // elementwise add: the first gradient is stored, a second one for the same tensor fails loudly.
  const Tensor& grad() const;
  void addGrad(Tensor&& g);
  void zeroGrad();

  void* rawPtr() const;
  template <typename T>
  T* dataPtr() const { return static_cast<T*>(rawPtr()); }

  void reshape_(const std::vector<int64_t>& shape);  // same element count; -1 for one inferred extent
  Tensor to(Device device) const;
  Tensor to(DType dtype) const;  // Float32 <-> Float16 / BFloat16, round to nearest even; done on the host
  Tensor clone() const;
  Tensor detach() const;  // the same storage without the autograd links (reference Tensor::detach)
  void fill_(float value);

  // Values as T on the host (Float32 / Float16 / BFloat16 / Bool / Int tensors are converted element-wise).
  template <typename T>
  std::vector<T> toList() const;

 private:
  struct Impl;
  std::shared_ptr<Impl> impl_;
  std::vector<float> toFloatList() const;
  void setFromFloats(const float* v, int64_t n);
};

// RNE conversions used by Tensor::to (same results as reference src/Utils/BFloat16.h:72-85, Half.h:226-257).
uint16_t floatToBFloat16Bits(float x);
float bfloat16BitsToFloat(uint16_t b);
uint16_t floatToHalfBits(float x);
float halfBitsToFloat(uint16_t b);

template <typename T>
Tensor::Tensor(const std::vector<T>& values, const std::vector<int64_t>& shape, Options options)
    : Tensor(shape, options) {
  ASSERT(static_cast<int64_t>(values.size()) == numel());
  std::vector<float> f(values.begin(), values.end());
  setFromFloats(f.data(), static_cast<int64_t>(f.size()));
}

template <typename T>
std::vector<T> Tensor::toList() const {
  std::vector<float> f = toFloatList();
  return std::vector<T>(f.begin(), f.end());
}

}  // namespace tinytorch
