// Tensor-level row-wise ops next to attention, declared with the reference's op names and signatures and registered
// for {GPU, Float32 / Float16 / BFloat16} the way the reference registers its device kernels
// (siluMul, fusedAddRmsNorm: src/Operation/OpFused.h:14-22, OpFusedCuda.cu:11-22; rmsNorm, softmax, logSoftmax:
// src/Operation/OpNNLayer.h:30-31,44,49,60-61).  Each GPU implementation is one call into the C ABI of
// include/ttfused.h on the thread's current stream.  The CPU slots are deliberately empty: a CPU tensor fails loudly
// through the dispatcher.
#pragma once

#include <vector>

#include "Dispatch.h"

namespace tinytorch::op {

// self [..., 2d] -> [..., d]: silu(self[..., :d]) * self[..., d:]
using SiluMulOpFn = Tensor (*)(const Tensor& self);
// in place: residual += input; input = rmsNorm(residual) * weight
using FusedAddRmsNormOpFn = void (*)(Tensor& input, Tensor& residual, const Tensor& weight, float eps);
// normalizedShape must be {self.size(-1)} (reference src/Operation/OpNNLayerCpu.h:183-184); weight may be undefined
using RMSNormOpFn = Tensor (*)(const Tensor& self, const std::vector<int64_t>& normalizedShape, const Tensor& weight,
                               float eps);
using SoftmaxOpFn = Tensor (*)(const Tensor& self, int64_t dim);

DEFINE_OP(siluMul, SiluMulOpFn)
DEFINE_OP(fusedAddRmsNorm, FusedAddRmsNormOpFn)
DEFINE_OP(rmsNorm, RMSNormOpFn)
DEFINE_OP(softmax, SoftmaxOpFn)
DEFINE_OP(logSoftmax, SoftmaxOpFn)
// gradient of softmax / logSoftmax along dim from the upstream gradient and the forward's output (reference
// src/Operation/OpNNLayer.h:46-51)
using SoftmaxOpBackwardFn = Tensor (*)(const Tensor& grad, const Tensor& output, int64_t dim);
DEFINE_OP(softmaxBackward, SoftmaxOpBackwardFn)
DEFINE_OP(logSoftmaxBackward, SoftmaxOpBackwardFn)

void registerFusedGpu();
STATIC_CALL(registerFusedGpu);

}  // namespace tinytorch::op
