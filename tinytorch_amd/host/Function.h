// Autograd-facing wrapper layer: Function<T>::apply, AutogradContext and the grad-mode switch, with the behaviour
// the attention path relies on (reference src/Tensor/Function.h:20-34,106-144, src/Tensor/NoGradGuard.h:11-34):
// when grad mode is on and an input requires grad, the output is marked and linked to a graph node that keeps the
// inputs; otherwise forward is a plain call with a null context.  Streams follow the reference's convention of one
// current stream per device and host thread (src/Utils/CUDAUtils.cpp:123-135).
#pragma once

#include <hip/hip_runtime.h>

#include <memory>
#include <type_traits>
#include <utility>
#include <vector>

#include "Tensor.h"

namespace tinytorch {

hipStream_t getCurrentStream(DeviceIndex device);
void synchronizeCurrentStream(DeviceIndex device);

class NoGradGuard {
 public:
  NoGradGuard() : prev_(gradEnabled) { gradEnabled = false; }
  ~NoGradGuard() { gradEnabled = prev_; }
  NoGradGuard(const NoGradGuard&) = delete;
  NoGradGuard& operator=(const NoGradGuard&) = delete;
  static bool isGradEnabled() { return gradEnabled; }

 private:
  static thread_local bool gradEnabled;
  bool prev_;
};

struct AutogradContext {
  explicit AutogradContext(std::vector<Tensor> inputs) : savedInputs(std::move(inputs)) {}
  std::vector<Tensor> savedInputs;
  std::vector<Tensor> savedForBackward;
  void saveForBackward(const Tensor& t) { savedForBackward.push_back(t); }
  // non-tensor arguments a backward needs (the reference keeps such values in an IValue list, src/Tensor/IValue.h)
  bool isCausal = false;
  float scale = 1.f;
  int64_t dim = -1;
};

struct FunctionBase {
  virtual ~FunctionBase() = default;
  virtual void backward(const Tensor& grad) = 0;
  std::vector<std::weak_ptr<FunctionBase>> nextFunctions;
};

template <class T>
class Function {
 public:
  struct Instance : FunctionBase {
    explicit Instance(std::shared_ptr<AutogradContext> c) : ctx(std::move(c)) {}
    void backward(const Tensor& grad) override { T::backward(ctx.get(), grad); }
    std::shared_ptr<AutogradContext> ctx;
  };

  template <typename... Args>
  static Tensor apply(Args&&... args) {
    bool requiresGrad = false;
    std::vector<Tensor> inputs;
    std::vector<std::weak_ptr<FunctionBase>> inputFns;
    if (NoGradGuard::isGradEnabled()) {
      auto visit = [&](auto&& arg) {
        using U = std::decay_t<decltype(arg)>;
        if constexpr (std::is_same_v<U, Tensor>) {
          if (arg.defined()) {
            requiresGrad = requiresGrad || arg.requiresGrad();
            inputs.push_back(arg);
            if (arg.gradFn()) inputFns.push_back(arg.gradFn());
          }
        }
      };
      (visit(args), ...);
    }
    auto ctx = requiresGrad ? std::make_shared<AutogradContext>(std::move(inputs)) : nullptr;
    Tensor out = T::forward(ctx.get(), std::forward<Args>(args)...);
    if (out.defined() && requiresGrad) {
      auto node = std::make_shared<Instance>(std::move(ctx));
      node->nextFunctions = std::move(inputFns);
      out.setRequiresGrad(true);
      out.setGradFn(node);
    }
    return out;
  }
};

}  // namespace tinytorch
