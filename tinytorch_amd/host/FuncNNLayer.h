// function::sdpAttention and its autograd wrapper, with the signature and defaults of the reference
// (src/Function/FuncNNLayer.h:229-268,298-302).  forward is a single op::sdpAttention call instead of the reference's
// matmul/transpose/scale/mask/softmax/matmul composite.  backward, NOT_IMPLEMENTED() in the reference (:267), is a
// single op::sdpAttentionBackward call that hands each input that requires grad its gradient with addGrad, the protocol
// of the reference's implemented backwards (src/Function/FuncActivation.h:53-61).
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
    const float scaleFactor =
        scale.has_value() ? scale.value() : (1.f / std::sqrt(static_cast<float>(query.size(-1))));
    Tensor out = op::sdpAttention(query, key, value, isCausal, attnMask, dropoutP, scaleFactor);
    if (ctx && out.defined()) {  // what backward needs beyond the saved inputs
      ctx->saveForBackward(out.detach());  // not `out` itself: it will own the node that owns this context
      ctx->saveForBackward(attnMask);
      ctx->isCausal = isCausal;
      ctx->scale = scaleFactor;
    }
    return out;
  }
  static void backward(AutogradContext* ctx, const Tensor& grad) {
    ASSERT(ctx && ctx->savedInputs.size() >= 3 && ctx->savedForBackward.size() == 2);
    if (!ctx || ctx->savedInputs.size() < 3 || ctx->savedForBackward.size() != 2) return;
    Tensor& query = ctx->savedInputs[0];
    Tensor& key = ctx->savedInputs[1];
    Tensor& value = ctx->savedInputs[2];
    auto grads = op::sdpAttentionBackward(grad, query, key, value, ctx->savedForBackward[0], ctx->isCausal,
                                          ctx->savedForBackward[1], ctx->scale);
    if (grads.size() != 3) return;
    if (query.requiresGrad()) query.addGrad(std::move(grads[0]));
    if (key.requiresGrad()) key.addGrad(std::move(grads[1]));
    if (value.requiresGrad()) value.addGrad(std::move(grads[2]));
  }
};

inline Tensor sdpAttention(const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal = false,
                           const Tensor& attnMask = {}, float dropoutP = 0.f,
                           std::optional<float> scale = std::nullopt) {
  return FuncSDPAttention::apply(query, key, value, isCausal, attnMask, dropoutP, scale);
}

}  // namespace tinytorch::function
