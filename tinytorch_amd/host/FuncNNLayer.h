// function::sdpAttention and its autograd wrapper, with the signature, defaults and backward behaviour of the
// reference (src/Function/FuncNNLayer.h:229-268,298-302).  forward is a single op::sdpAttention call instead of the
// reference's matmul/transpose/scale/mask/softmax/matmul composite; backward is not implemented there either (:267).
#pragma once

#include <cmath>
#include <optional>

#include "Function.h"
#include "OpAttention.h"

namespace tinytorch::function {

class FuncSDPAttention : public Function<FuncSDPAttention> {
 public:
  static Tensor forward(AutogradContext* ctx, const Tensor& query, const Tensor& key, const Tensor& value,
                        bool isCausal, const Tensor& attnMask, float dropoutP, std::optional<float> scale) {
    (void)ctx;
    const float scaleFactor =
        scale.has_value() ? scale.value() : (1.f / std::sqrt(static_cast<float>(query.size(-1))));
    return op::sdpAttention(query, key, value, isCausal, attnMask, dropoutP, scaleFactor);
  }
  static void backward(AutogradContext* ctx, const Tensor& grad) {
    (void)ctx;
    (void)grad;
    NOT_IMPLEMENTED();
  }
};

inline Tensor sdpAttention(const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal = false,
                           const Tensor& attnMask = {}, float dropoutP = 0.f,
                           std::optional<float> scale = std::nullopt) {
  return FuncSDPAttention::apply(query, key, value, isCausal, attnMask, dropoutP, scale);
}

}  // namespace tinytorch::function
