// function::siluMul / fusedAddRmsNorm / rmsNorm / softmax / logSoftmax with the reference's signatures and defaults
// (src/Function/FuncFused.h:14-34, src/Function/FuncNNLayer.h:219-227,294-296, src/Function/FuncActivation.h:42-92).
// Forward only: the reference's backward of siluMul, fusedAddRmsNorm and rmsNorm is NOT_IMPLEMENTED as well; the
// softmax / logSoftmax backward is the reference's own (op::softmaxBackward / op::logSoftmaxBackward).
#pragma once

#include <vector>

#include "Function.h"
#include "OpFused.h"
#include "OpLinalg.h"

namespace tinytorch::function {

class FuncSiluMul : public Function<FuncSiluMul> {
 public:
  static Tensor forward(AutogradContext* ctx, const Tensor& x) {
    (void)ctx;
    return op::siluMul(x);
  }
  static void backward(AutogradContext* ctx, const Tensor& grad) {
    (void)ctx, (void)grad;
    NOT_IMPLEMENTED();
  }
};

class FuncRMSNorm : public Function<FuncRMSNorm> {
 public:
  static Tensor forward(AutogradContext* ctx, const Tensor& input, const std::vector<int64_t>& normalizedShape,
                        const Tensor& weight, float eps) {
    (void)ctx;
    return op::rmsNorm(input, normalizedShape, weight, eps);
  }
  static void backward(AutogradContext* ctx, const Tensor& grad) {
    (void)ctx, (void)grad;
    NOT_IMPLEMENTED();
  }
};

template <bool LOG>
class FuncSoftmaxT : public Function<FuncSoftmaxT<LOG>> {
 public:
  // forward keeps its output and the axis; backward is the reference's (src/Function/FuncActivation.h:45-62, 68-85)
  static Tensor forward(AutogradContext* ctx, const Tensor& self, int64_t dim) {
    Tensor out = LOG ? op::logSoftmax(self, dim) : op::softmax(self, dim);
    if (ctx && out.defined()) {
      ctx->saveForBackward(out.detach());
      ctx->dim = dim;
    }
    return out;
  }
  static void backward(AutogradContext* ctx, const Tensor& grad) {
    ASSERT(ctx && !ctx->savedInputs.empty() && ctx->savedForBackward.size() == 1);
    if (!ctx || ctx->savedInputs.empty() || ctx->savedForBackward.size() != 1) return;
    Tensor& self = ctx->savedInputs[0];
    if (self.requiresGrad()) {
      const Tensor& output = ctx->savedForBackward[0];
      self.addGrad(LOG ? op::logSoftmaxBackward(grad, output, ctx->dim) : op::softmaxBackward(grad, output, ctx->dim));
    }
  }
};

// function::linear (reference src/Function/FuncNNLayer.h:14-36, 270-272): forward is the reference's single op call,
// backward its three: grad . weight, grad^T . input and the column sums of grad (here: ones[1, M] . grad, this layer
// having no reduction op).
class FuncLinear : public Function<FuncLinear> {
 public:
  static Tensor forward(AutogradContext* ctx, const Tensor& input, const Tensor& weight, const Tensor& bias) {
    (void)ctx;
    return op::matmul(input, weight, false, true, bias);
  }
  static void backward(AutogradContext* ctx, const Tensor& grad) {
    ASSERT(ctx && ctx->savedInputs.size() >= 2);
    if (!ctx || ctx->savedInputs.size() < 2) return;
    Tensor& input = ctx->savedInputs[0];
    Tensor& weight = ctx->savedInputs[1];
    if (input.requiresGrad()) input.addGrad(op::matmul(grad, weight, false, false, Tensor{}));
    const int64_t N = weight.size(0), K = weight.size(1);
    Tensor g2 = grad.detach(), x2 = input.detach();  // [M, N] and [M, K] views of the same storage
    g2.reshape_({-1, N});
    x2.reshape_({-1, K});
    if (weight.requiresGrad()) weight.addGrad(op::matmul(g2, x2, true, false, Tensor{}));
    if (ctx->savedInputs.size() > 2 && ctx->savedInputs[2].requiresGrad()) {
      Tensor ones = Tensor::ones({1, g2.size(0)}, g2.options().noGrad());
      Tensor gb = op::matmul(ones, g2, false, false, Tensor{});
      gb.reshape_({N});
      ctx->savedInputs[2].addGrad(std::move(gb));
    }
  }
};

inline Tensor linear(const Tensor& input, const Tensor& weight, const Tensor& bias = {}) {
  return FuncLinear::apply(input, weight, bias);
}

inline Tensor siluMul(const Tensor& x) { return FuncSiluMul::apply(x); }

// In place on input and residual; no autograd node (the reference's wrapper has none to offer either: its backward is
// NOT_IMPLEMENTED, src/Function/FuncFused.h:27).
inline void fusedAddRmsNorm(Tensor& input, Tensor& residual, const Tensor& weight, float eps) {
  op::fusedAddRmsNorm(input, residual, weight, eps);
}

inline Tensor rmsNorm(const Tensor& input, const std::vector<int64_t>& normalizedShape, const Tensor& weight,
                      float eps = 1e-8f) {
  return FuncRMSNorm::apply(input, normalizedShape, weight, eps);
}

inline Tensor softmax(const Tensor& self, int64_t dim = -1) { return FuncSoftmaxT<false>::apply(self, dim); }
inline Tensor logSoftmax(const Tensor& self, int64_t dim = -1) { return FuncSoftmaxT<true>::apply(self, dim); }

}  // namespace tinytorch::function
