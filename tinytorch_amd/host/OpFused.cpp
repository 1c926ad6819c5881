// GPU implementations of the row-wise ops: argument checks in the reference's style (ASSERT, then a defined failure
// value), one enqueue through include/ttfused.h, outputs from the caching allocator, no host synchronisation.
#include "OpFused.h"

#include "../../include/ttfused.h"
#include "Function.h"
#include "Macros.h"

namespace tinytorch::op {

namespace {

int dtypeCode(DType t) {
  switch (t) {
    case DType::Float32: return TTSDPA_F32;
    case DType::Float16: return TTSDPA_F16;
    default: return TTSDPA_BF16;
  }
}

hipStream_t streamOf(const Tensor& t) {
  const DeviceIndex dev = t.device().index;
  HIP_CHECK(hipSetDevice(dev));
  return getCurrentStream(dev);
}

bool launched(const char* what, int rc) {
  if (rc != TTSDPA_OK) {
    LOGE("%s failed: %d (%s)", what, rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return false;
  }
  return true;
}

Tensor siluMulGpuImpl(const Tensor& self) {
  ASSERT(self.defined() && self.dim() >= 1 && self.size(-1) % 2 == 0);  // reference src/Operation/OpFusedCuda.cuh:68
  if (!self.defined() || self.dim() < 1 || self.size(-1) % 2 != 0) return {};
  std::vector<int64_t> shape = self.shape();
  shape.back() /= 2;
  Tensor out = Tensor::empty(shape, self.options().noGrad());
  const int64_t d = shape.back();
  const int64_t rows = d ? out.numel() / d : 0;
  if (!launched("ttfused_silu_mul", ttfused_silu_mul(dtypeCode(self.dtype()), self.rawPtr(), out.rawPtr(), rows, d, streamOf(self))))
    return {};
  return out;
}

void fusedAddRmsNormGpuImpl(Tensor& input, Tensor& residual, const Tensor& weight, float eps) {
  ASSERT(input.defined() && residual.defined() && weight.defined());
  ASSERT(input.shape() == residual.shape());  // reference src/Operation/OpFusedCuda.cuh:131
  ASSERT(residual.dtype() == input.dtype() && weight.dtype() == input.dtype());
  ASSERT(residual.device() == input.device() && weight.device() == input.device());
  if (!input.defined() || !residual.defined() || !weight.defined() || input.shape() != residual.shape() || input.dim() < 1) return;
  const int64_t dim = input.size(-1);
  ASSERT(weight.numel() == dim);
  if (weight.numel() != dim) return;
  const int64_t rows = dim ? input.numel() / dim : 0;
  launched("ttfused_add_rms_norm", ttfused_add_rms_norm(dtypeCode(input.dtype()), input.rawPtr(), residual.rawPtr(),
                                                        weight.rawPtr(), rows, dim, eps, streamOf(input)));
}

Tensor rmsNormGpuImpl(const Tensor& self, const std::vector<int64_t>& normalizedShape, const Tensor& weight, float eps) {
  ASSERT(self.defined() && self.dim() >= 1);
  if (!self.defined() || self.dim() < 1) return {};
  const int64_t dim = self.size(-1);
  ASSERT(normalizedShape.size() == 1 && normalizedShape.front() == dim);  // reference src/Operation/OpNNLayerCuda.cuh:491-492
  if (normalizedShape.size() != 1 || normalizedShape.front() != dim) return {};
  if (weight.defined()) {
    ASSERT(weight.numel() == dim && weight.dtype() == self.dtype() && weight.device() == self.device());
    if (weight.numel() != dim || weight.dtype() != self.dtype()) return {};
  }
  Tensor out = Tensor::empty(self.shape(), self.options().noGrad());
  const int64_t rows = dim ? self.numel() / dim : 0;
  if (!launched("ttfused_rms_norm", ttfused_rms_norm(dtypeCode(self.dtype()), self.rawPtr(), weight.defined() ? weight.rawPtr() : nullptr,
                                                     out.rawPtr(), rows, dim, eps, streamOf(self))))
    return {};
  return out;
}

template <bool LOG>
Tensor softmaxGpuImpl(const Tensor& self, int64_t dim) {
  ASSERT(self.defined() && self.dim() >= 1);
  if (!self.defined() || self.dim() < 1) return {};
  if (dim < 0) dim += self.dim();
  ASSERT(dim >= 0 && dim < self.dim());
  if (dim < 0 || dim >= self.dim()) return {};
  int64_t outer = 1, inner = 1;  // reference getSoftmaxDimInfo, src/Operation/OpNNLayer.h:22-29
  for (int64_t i = 0; i < dim; i++) outer *= self.size(i);
  for (int64_t i = dim + 1; i < self.dim(); i++) inner *= self.size(i);
  Tensor out = Tensor::empty(self.shape(), self.options().noGrad());
  if (!launched("ttfused_softmax", ttfused_softmax(dtypeCode(self.dtype()), self.rawPtr(), out.rawPtr(), outer, self.size(dim), inner,
                                                   LOG ? 1 : 0, streamOf(self))))
    return {};
  return out;
}

template <bool LOG>
Tensor softmaxBackwardGpuImpl(const Tensor& grad, const Tensor& output, int64_t dim) {
  ASSERT(grad.defined() && output.defined() && output.shape() == grad.shape() && output.dtype() == grad.dtype());
  if (!grad.defined() || !output.defined() || output.shape() != grad.shape() || output.dtype() != grad.dtype() || grad.dim() < 1) return {};
  if (dim < 0) dim += grad.dim();
  ASSERT(dim >= 0 && dim < grad.dim());
  if (dim < 0 || dim >= grad.dim()) return {};
  int64_t outer = 1, inner = 1;
  for (int64_t i = 0; i < dim; i++) outer *= grad.size(i);
  for (int64_t i = dim + 1; i < grad.dim(); i++) inner *= grad.size(i);
  Tensor out = Tensor::empty(grad.shape(), grad.options().noGrad());
  if (!launched("ttfused_softmax_backward",
                ttfused_softmax_backward(dtypeCode(grad.dtype()), grad.rawPtr(), output.rawPtr(), out.rawPtr(), outer, grad.size(dim),
                                         inner, LOG ? 1 : 0, streamOf(grad))))
    return {};
  return out;
}

}  // namespace

void registerFusedGpu() {
  REGISTER_OP_IMPL(siluMul, GPU, Float32, &siluMulGpuImpl);
  REGISTER_OP_IMPL(siluMul, GPU, Float16, &siluMulGpuImpl);
  REGISTER_OP_IMPL(siluMul, GPU, BFloat16, &siluMulGpuImpl);
  REGISTER_OP_IMPL(fusedAddRmsNorm, GPU, Float32, &fusedAddRmsNormGpuImpl);
  REGISTER_OP_IMPL(fusedAddRmsNorm, GPU, Float16, &fusedAddRmsNormGpuImpl);
  REGISTER_OP_IMPL(fusedAddRmsNorm, GPU, BFloat16, &fusedAddRmsNormGpuImpl);
  REGISTER_OP_IMPL(rmsNorm, GPU, Float32, &rmsNormGpuImpl);
  REGISTER_OP_IMPL(rmsNorm, GPU, Float16, &rmsNormGpuImpl);
  REGISTER_OP_IMPL(rmsNorm, GPU, BFloat16, &rmsNormGpuImpl);
  REGISTER_OP_IMPL(softmax, GPU, Float32, &softmaxGpuImpl<false>);
  REGISTER_OP_IMPL(softmax, GPU, Float16, &softmaxGpuImpl<false>);
  REGISTER_OP_IMPL(softmax, GPU, BFloat16, &softmaxGpuImpl<false>);
  REGISTER_OP_IMPL(logSoftmax, GPU, Float32, &softmaxGpuImpl<true>);
  REGISTER_OP_IMPL(logSoftmax, GPU, Float16, &softmaxGpuImpl<true>);
  REGISTER_OP_IMPL(logSoftmax, GPU, BFloat16, &softmaxGpuImpl<true>);
  REGISTER_OP_IMPL(softmaxBackward, GPU, Float32, &softmaxBackwardGpuImpl<false>);
  REGISTER_OP_IMPL(softmaxBackward, GPU, Float16, &softmaxBackwardGpuImpl<false>);
  REGISTER_OP_IMPL(softmaxBackward, GPU, BFloat16, &softmaxBackwardGpuImpl<false>);
  REGISTER_OP_IMPL(logSoftmaxBackward, GPU, Float32, &softmaxBackwardGpuImpl<true>);
  REGISTER_OP_IMPL(logSoftmaxBackward, GPU, Float16, &softmaxBackwardGpuImpl<true>);
  REGISTER_OP_IMPL(logSoftmaxBackward, GPU, BFloat16, &softmaxBackwardGpuImpl<true>);
}

}  // namespace tinytorch::op
