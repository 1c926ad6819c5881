#include "OpLinalg.h"

#include "../../include/ttlinear.h"
#include "Function.h"
#include "Macros.h"

namespace tinytorch::op {

namespace {

Tensor matmulGpuImpl(const Tensor& a, const Tensor& b, bool transA, bool transB, const Tensor& bias) {
  ASSERT(a.defined() && b.defined());
  ASSERT(!transA && transB);  // the linear layer's call; the reference's other flag combinations are not built here
  ASSERT(a.dim() >= 1 && b.dim() == 2 && a.size(-1) == b.size(1));
  ASSERT(b.dtype() == a.dtype() && b.device() == a.device());
  if (!a.defined() || !b.defined() || transA || !transB || a.dim() < 1 || b.dim() != 2 || a.size(-1) != b.size(1) ||
      b.dtype() != a.dtype())
    return {};
  const int64_t K = b.size(1), N = b.size(0);
  if (bias.defined()) {
    ASSERT(bias.dim() == 1 && bias.size(0) == N && bias.dtype() == a.dtype());  // reference src/Operation/OpLinalg.cpp:262
    if (bias.dim() != 1 || bias.size(0) != N || bias.dtype() != a.dtype()) return {};
  }
  std::vector<int64_t> shape = a.shape();
  shape.back() = N;
  int64_t M = 1;
  for (size_t i = 0; i + 1 < shape.size(); i++) M *= shape[i];
  Tensor out = Tensor::empty(shape, a.options().noGrad());
  const int dtype = a.dtype() == DType::Float32 ? TTSDPA_F32 : a.dtype() == DType::Float16 ? TTSDPA_F16 : TTSDPA_BF16;
  const DeviceIndex dev = a.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const int rc = ttlinear_forward(dtype, a.rawPtr(), b.rawPtr(), bias.defined() ? bias.rawPtr() : nullptr, out.rawPtr(), M, N, K,
                                  K, K, N, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttlinear_forward failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  return out;
}

}  // namespace

void registerLinalgGpu() {
  REGISTER_OP_IMPL(matmul, GPU, Float32, &matmulGpuImpl);
  REGISTER_OP_IMPL(matmul, GPU, Float16, &matmulGpuImpl);
  REGISTER_OP_IMPL(matmul, GPU, BFloat16, &matmulGpuImpl);
}

}  // namespace tinytorch::op
