#include "Tensor.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <map>
#include <mutex>

#include "Function.h"

namespace tinytorch {

// ---- logging / assertions ----------------------------------------------------------------------------------------

namespace {
LogFunc g_logFunc = nullptr;
AssertHandler g_assertHandler = nullptr;
std::mutex g_logMutex;
}  // namespace

void setLogFunc(LogFunc fn) { g_logFunc = fn; }

void logMessage(int level, const char* file, int line, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  std::lock_guard<std::mutex> lock(g_logMutex);
  if (g_logFunc) {
    g_logFunc(level, buf);
    return;
  }
  static const char* names[] = {"INFO", "DEBUG", "WARN", "ERROR"};
  std::FILE* out = level >= 2 ? stderr : stdout;
  std::fprintf(out, "[TinyTorch][%s] %s:%d: %s\n", names[level & 3], file, line, buf);
  std::fflush(out);
}

AssertHandler setAssertHandler(AssertHandler h) {
  AssertHandler old = g_assertHandler;
  g_assertHandler = h;
  return old;
}

void assertFailed(const char* expr, const char* file, int line) {
  if (g_assertHandler) {
    g_assertHandler(expr, file, line);
    return;
  }
  __builtin_trap();
}

// ---- dtype / device ------------------------------------------------------------------------------------------------

size_t dtypeSize(DType t) {
  switch (t) {
    case DType::Float32: return 4;
    case DType::Float16: return 2;
    case DType::BFloat16: return 2;
    case DType::Int32: return 4;
    case DType::Int64: return 8;
    case DType::Bool: return 1;
    default: return 0;
  }
}

const char* dtypeToString(DType t) {
  switch (t) {
    case DType::Float32: return "Float32";
    case DType::Float16: return "Float16";
    case DType::BFloat16: return "BFloat16";
    case DType::Int32: return "Int32";
    case DType::Int64: return "Int64";
    case DType::Bool: return "Bool";
    default: return "Unknown";
  }
}

const char* deviceTypeToString(DeviceType t) { return t == DeviceType::CPU ? "CPU" : "GPU"; }

namespace {
Device g_defaultDevice;
}
void setDefaultDevice(Device d) { g_defaultDevice = d; }
Device getDefaultDevice() { return g_defaultDevice; }

// ---- 16-bit conversions ---------------------------------------------------------------------------------------------

uint16_t floatToBFloat16Bits(float x) {
  uint32_t u;
  std::memcpy(&u, &x, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  return static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
float bfloat16BitsToFloat(uint16_t b) {
  uint32_t u = static_cast<uint32_t>(b) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
uint16_t floatToHalfBits(float x) {
  // IEEE binary16, round to nearest even; NaN -> sign | 0x7E00
  uint32_t u;
  std::memcpy(&u, &x, 4);
  const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
  const uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return static_cast<uint16_t>(sign | 0x7E00u);
  if (mag >= 0x47800000u) return static_cast<uint16_t>(sign | 0x7C00u);  // 65536 and above (incl. inf)
  const int e = static_cast<int>(mag >> 23) - 127;
  const uint32_t man = mag & 0x7FFFFFu;
  if (e < -25) return sign;
  uint32_t q, rem, half;
  if (e < -14) {  // subnormal half: units of 2^-24
    const uint32_t full = man | 0x800000u;
    const int shift = -e - 1;
    q = full >> shift;
    rem = full & ((1u << shift) - 1u);
    half = 1u << (shift - 1);
  } else {
    q = (static_cast<uint32_t>(e + 15) << 10) | (man >> 13);
    rem = man & 0x1FFFu;
    half = 0x1000u;
  }
  if (rem > half || (rem == half && (q & 1u))) q++;
  return static_cast<uint16_t>(sign | q);
}
float halfBitsToFloat(uint16_t b) {
  const uint32_t sign = (static_cast<uint32_t>(b) & 0x8000u) << 16;
  const uint32_t e = (b >> 10) & 0x1Fu, m = b & 0x3FFu;
  uint32_t u;
  if (e == 0x1F) {
    u = sign | 0x7F800000u | (m << 13);
  } else if (e == 0) {
    if (m == 0) {
      u = sign;
    } else {
      float f = static_cast<float>(m) * 5.9604644775390625e-08f;  // m * 2^-24, exact
      std::memcpy(&u, &f, 4);
      u |= sign;
    }
  } else {
    u = sign | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// ---- device allocator --------------------------------------------------------------------------------------------------

namespace {

// Free blocks are kept by rounded size and handed out again without going back to hipMalloc.  Everything on this
// path runs on one stream per device and thread, so a block freed on the host can be reused by the next enqueue.
struct DeviceCache {
  std::mutex mutex;
  std::multimap<size_t, void*> freeBlocks;
  std::map<void*, size_t> live;
  size_t cachedBytes = 0, liveBytes = 0;
};
DeviceCache& cacheOf(DeviceIndex d) {
  static DeviceCache caches[16];
  return caches[d & 15];
}
size_t roundUp(size_t n) { return n == 0 ? 512 : (n + 511) / 512 * 512; }

void* deviceAlloc(DeviceIndex dev, size_t nbytes) {
  size_t need = roundUp(nbytes);
  DeviceCache& c = cacheOf(dev);
  std::lock_guard<std::mutex> lock(c.mutex);
  auto it = c.freeBlocks.lower_bound(need);
  void* p = nullptr;
  size_t got = need;
  if (it != c.freeBlocks.end() && it->first <= 2 * need) {
    p = it->second;
    got = it->first;
    c.cachedBytes -= got;
    c.freeBlocks.erase(it);
  } else {
    HIP_CHECK(hipSetDevice(dev));
    HIP_CHECK(hipMalloc(&p, need));
  }
  c.live[p] = got;
  c.liveBytes += got;
  return p;
}

void deviceFree(DeviceIndex dev, void* p) {
  if (!p) return;
  DeviceCache& c = cacheOf(dev);
  std::lock_guard<std::mutex> lock(c.mutex);
  auto it = c.live.find(p);
  ASSERT(it != c.live.end());
  if (it == c.live.end()) return;
  c.freeBlocks.emplace(it->second, p);
  c.cachedBytes += it->second;
  c.liveBytes -= it->second;
  c.live.erase(it);
}

}  // namespace

size_t deviceAllocatorCachedBytes(DeviceIndex device) { return cacheOf(device).cachedBytes; }
size_t deviceAllocatorLiveBytes(DeviceIndex device) { return cacheOf(device).liveBytes; }
void deviceAllocatorRelease(DeviceIndex device) {
  DeviceCache& c = cacheOf(device);
  std::lock_guard<std::mutex> lock(c.mutex);
  HIP_CHECK(hipSetDevice(device));
  HIP_CHECK(hipDeviceSynchronize());
  for (auto& kv : c.freeBlocks) HIP_CHECK(hipFree(kv.second));
  c.freeBlocks.clear();
  c.cachedBytes = 0;
}

// ---- storage -----------------------------------------------------------------------------------------------------------

Storage::Storage(size_t nbytes, Device device) : nbytes_(nbytes), device_(device) {
  if (device.isCpu()) {
    data_ = std::aligned_alloc(64, roundUp(nbytes));
    ASSERT(data_ != nullptr);
  } else {
    data_ = deviceAlloc(device.index, nbytes);
  }
}

Storage::~Storage() {
  if (device_.isCpu()) {
    std::free(data_);
  } else {
    deviceFree(device_.index, data_);
  }
}

void Storage::copy(void* dst, Device dstDev, const void* src, Device srcDev, size_t nbytes) {
  if (nbytes == 0) return;
  if (dstDev.isCpu() && srcDev.isCpu()) {
    std::memcpy(dst, src, nbytes);
    return;
  }
  Device gpu = dstDev.isGpu() ? dstDev : srcDev;
  HIP_CHECK(hipSetDevice(gpu.index));
  hipStream_t stream = getCurrentStream(gpu.index);
  hipMemcpyKind kind = dstDev.isCpu() ? hipMemcpyDeviceToHost : (srcDev.isCpu() ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice);
  HIP_CHECK(hipMemcpyAsync(dst, src, nbytes, kind, stream));
  // transfers that touch host memory complete before returning, as in the reference (src/Tensor/Storage.cpp:65-76)
  if (kind != hipMemcpyDeviceToDevice) HIP_CHECK(hipStreamSynchronize(stream));
}

// ---- streams -------------------------------------------------------------------------------------------------------------

hipStream_t getCurrentStream(DeviceIndex device) {
  // one lazily created stream per device and host thread (reference src/Utils/CUDAUtils.cpp:123-135)
  thread_local hipStream_t streams[16] = {};
  hipStream_t& s = streams[device & 15];
  if (!s) {
    HIP_CHECK(hipSetDevice(device));
    HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  }
  return s;
}

void synchronizeCurrentStream(DeviceIndex device) { HIP_CHECK(hipStreamSynchronize(getCurrentStream(device))); }

// ---- tensor ----------------------------------------------------------------------------------------------------------------

struct Tensor::Impl {
  std::vector<int64_t> shape;
  int64_t numel = 1;
  Options options;
  std::shared_ptr<Storage> storage;
  std::shared_ptr<FunctionBase> gradFn;
  Tensor grad;
};

Tensor::Tensor(const std::vector<int64_t>& shape, Options options) {
  impl_ = std::make_shared<Impl>();
  impl_->shape = shape;
  impl_->numel = 1;
  for (int64_t s : shape) {
    ASSERT(s >= 0);
    impl_->numel *= s;
  }
  impl_->options = options;
  impl_->storage = std::make_shared<Storage>(static_cast<size_t>(impl_->numel) * dtypeSize(options.dtype_), options.device_);
}

const std::vector<int64_t>& Tensor::shape() const {
  static const std::vector<int64_t> empty;
  return impl_ ? impl_->shape : empty;
}
int64_t Tensor::size(int64_t d) const {
  int64_t n = dim();
  if (d < 0) d += n;
  ASSERT(d >= 0 && d < n);
  return impl_->shape[static_cast<size_t>(d)];
}
int64_t Tensor::numel() const { return impl_ ? impl_->numel : 0; }
DType Tensor::dtype() const { return impl_->options.dtype_; }
Device Tensor::device() const { return impl_->options.device_; }
Options Tensor::options() const { return impl_->options; }
bool Tensor::requiresGrad() const { return impl_ && impl_->options.requiresGrad_; }
void Tensor::setRequiresGrad(bool r) { impl_->options.requiresGrad_ = r; }
std::shared_ptr<FunctionBase> Tensor::gradFn() const { return impl_ ? impl_->gradFn : nullptr; }
void Tensor::setGradFn(std::shared_ptr<FunctionBase> fn) { impl_->gradFn = std::move(fn); }
const Tensor& Tensor::grad() const {
  static const Tensor none;
  return impl_ ? impl_->grad : none;
}
void Tensor::addGrad(Tensor&& g) {
  ASSERT(impl_ && requiresGrad());
  ASSERT(!impl_->grad.defined());  // accumulation needs an elementwise add, which this layer does not carry
  if (impl_ && !impl_->grad.defined()) impl_->grad = std::move(g);
}
Tensor Tensor::detach() const {
  Tensor t;
  if (impl_) {
    t.impl_ = std::make_shared<Impl>();
    t.impl_->shape = impl_->shape;
    t.impl_->numel = impl_->numel;
    t.impl_->options = impl_->options.noGrad();
    t.impl_->storage = impl_->storage;
  }
  return t;
}
void Tensor::zeroGrad() {
  if (impl_) impl_->grad = Tensor();
}
void* Tensor::rawPtr() const { return impl_->storage->data(); }

void Tensor::reshape_(const std::vector<int64_t>& shape) {
  std::vector<int64_t> s = shape;
  int64_t known = 1, infer = -1;
  for (size_t i = 0; i < s.size(); i++) {
    if (s[i] == -1) {
      ASSERT(infer < 0);
      infer = static_cast<int64_t>(i);
    } else {
      known *= s[i];
    }
  }
  if (infer >= 0) s[static_cast<size_t>(infer)] = known ? impl_->numel / known : 0;
  int64_t n = 1;
  for (int64_t v : s) n *= v;
  ASSERT(n == impl_->numel);
  impl_->shape = s;
}

Tensor Tensor::to(Device device) const {
  if (device == this->device()) return *this;
  Tensor out(shape(), options().noGrad().device(device));
  Storage::copy(out.rawPtr(), device, rawPtr(), this->device(), static_cast<size_t>(numel()) * dtypeSize(dtype()));
  return out;
}

Tensor Tensor::clone() const {
  Tensor out(shape(), options().noGrad());
  Storage::copy(out.rawPtr(), device(), rawPtr(), device(), static_cast<size_t>(numel()) * dtypeSize(dtype()));
  return out;
}

std::vector<float> Tensor::toFloatList() const {
  Tensor h = to(Device(DeviceType::CPU));
  int64_t n = numel();
  std::vector<float> out(static_cast<size_t>(n));
  switch (dtype()) {
    case DType::Float32: std::memcpy(out.data(), h.rawPtr(), static_cast<size_t>(n) * 4); break;
    case DType::Float16:
      for (int64_t i = 0; i < n; i++) out[i] = halfBitsToFloat(h.dataPtr<uint16_t>()[i]);
      break;
    case DType::BFloat16:
      for (int64_t i = 0; i < n; i++) out[i] = bfloat16BitsToFloat(h.dataPtr<uint16_t>()[i]);
      break;
    case DType::Int32:
      for (int64_t i = 0; i < n; i++) out[i] = static_cast<float>(h.dataPtr<int32_t>()[i]);
      break;
    case DType::Int64:
      for (int64_t i = 0; i < n; i++) out[i] = static_cast<float>(h.dataPtr<int64_t>()[i]);
      break;
    case DType::Bool:
      for (int64_t i = 0; i < n; i++) out[i] = h.dataPtr<uint8_t>()[i] ? 1.f : 0.f;
      break;
    default: ASSERT(!"unsupported dtype");
  }
  return out;
}

void Tensor::setFromFloats(const float* v, int64_t n) {
  ASSERT(n == numel());
  size_t bytes = static_cast<size_t>(n) * dtypeSize(dtype());
  std::vector<uint8_t> staging(bytes ? bytes : 1);
  switch (dtype()) {
    case DType::Float32: std::memcpy(staging.data(), v, bytes); break;
    case DType::Float16:
      for (int64_t i = 0; i < n; i++) reinterpret_cast<uint16_t*>(staging.data())[i] = floatToHalfBits(v[i]);
      break;
    case DType::BFloat16:
      for (int64_t i = 0; i < n; i++) reinterpret_cast<uint16_t*>(staging.data())[i] = floatToBFloat16Bits(v[i]);
      break;
    case DType::Int32:
      for (int64_t i = 0; i < n; i++) reinterpret_cast<int32_t*>(staging.data())[i] = static_cast<int32_t>(v[i]);
      break;
    case DType::Int64:
      for (int64_t i = 0; i < n; i++) reinterpret_cast<int64_t*>(staging.data())[i] = static_cast<int64_t>(v[i]);
      break;
    case DType::Bool:
      for (int64_t i = 0; i < n; i++) staging[i] = v[i] != 0.f;
      break;
    default: ASSERT(!"unsupported dtype");
  }
  Storage::copy(rawPtr(), device(), staging.data(), Device(DeviceType::CPU), bytes);
}

Tensor Tensor::to(DType t) const {
  if (t == dtype()) return *this;
  std::vector<float> f = toFloatList();
  Tensor out(shape(), options().noGrad().dtype(t));
  out.setFromFloats(f.data(), static_cast<int64_t>(f.size()));
  return out;
}

void Tensor::fill_(float value) {
  std::vector<float> f(static_cast<size_t>(numel()), value);
  setFromFloats(f.data(), numel());
}

Tensor Tensor::zeros(const std::vector<int64_t>& shape, Options options) {
  Tensor t(shape, options);
  t.fill_(0.f);
  return t;
}
Tensor Tensor::ones(const std::vector<int64_t>& shape, Options options) {
  Tensor t(shape, options);
  t.fill_(1.f);
  return t;
}
Tensor Tensor::scalar(float value, Options options) {
  Tensor t({}, options);
  t.fill_(value);
  return t;
}

// ---- grad mode ---------------------------------------------------------------------------------------------------------------

thread_local bool NoGradGuard::gradEnabled = true;

}  // namespace tinytorch
