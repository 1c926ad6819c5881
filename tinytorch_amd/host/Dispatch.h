// {device, dtype} -> function-pointer dispatch for Tensor-level ops, with the table layout and the registration
// macros of the reference (src/Tensor/Dispatch.h:21-48,59-94,110-142): table[device * DTypeCount + dtype], filled
// by idempotent registration functions during static initialisation, read-only afterwards.  A missing entry is a
// loud failure (message on stderr + ASSERT), never a silent fallback.
#pragma once

#include <cstddef>
#include <iostream>
#include <string>
#include <type_traits>
#include <utility>

#include "Tensor.h"

namespace tinytorch {

struct DispatchKey {
  DeviceType device;
  DType dtype;
  std::string toString() const {
    return std::string("{ device: ") + deviceTypeToString(device) + ", dtype: " + dtypeToString(dtype) + "}";
  }
};

constexpr size_t dispatchKeyToIndex(DispatchKey k) {
  return static_cast<size_t>(k.device) * static_cast<size_t>(DType::DTypeCount) + static_cast<size_t>(k.dtype);
}
constexpr size_t NumDispatchKeys =
    static_cast<size_t>(DeviceType::DeviceTypeCount) * static_cast<size_t>(DType::DTypeCount);

template <typename Tag, typename Fn>
struct OpRegistry {
  static Fn table[NumDispatchKeys];
  static void registerImpl(DispatchKey key, Fn fn) { table[dispatchKeyToIndex(key)] = fn; }
  static Fn lookup(DispatchKey key) { return table[dispatchKeyToIndex(key)]; }
};
template <typename Tag, typename Fn>
Fn OpRegistry<Tag, Fn>::table[NumDispatchKeys] = {nullptr};

// The key comes from the first Tensor (or Options) among the arguments.
inline DispatchKey dispatchKeyOf(const Tensor& t) { return {t.device().type, t.dtype()}; }
inline DispatchKey dispatchKeyOf(const Options& o) { return {o.device_.type, o.dtype_}; }

template <typename First, typename... Rest>
DispatchKey getDispatchKeyFromArgs(First&& first, Rest&&... rest) {
  using U = std::decay_t<First>;
  if constexpr (std::is_same_v<U, Tensor> || std::is_same_v<U, Options>) {
    return dispatchKeyOf(first);
  } else {
    static_assert(sizeof...(Rest) > 0, "op call without a Tensor or Options argument");
    return getDispatchKeyFromArgs(std::forward<Rest>(rest)...);
  }
}

}  // namespace tinytorch

#define DEFINE_OP(NAME, FN_TYPE)                                                                   \
  struct NAME##_op_tag {};                                                                         \
  using NAME##_registry = ::tinytorch::OpRegistry<NAME##_op_tag, FN_TYPE>;                         \
  template <typename... Args>                                                                      \
  auto NAME(Args&&... args) -> std::invoke_result_t<FN_TYPE, Args...> {                            \
    ::tinytorch::DispatchKey key = ::tinytorch::getDispatchKeyFromArgs(args...);                   \
    FN_TYPE fn = NAME##_registry::lookup(key);                                                     \
    if (!fn) {                                                                                     \
      std::cerr << "op " #NAME ": no implementation registered for " << key.toString() << std::endl; \
      ASSERT(fn != nullptr);                                                                       \
      return std::invoke_result_t<FN_TYPE, Args...>();                                             \
    }                                                                                              \
    return fn(std::forward<Args>(args)...);                                                        \
  }

#define REGISTER_OP_IMPL(NAME, DEVICE, DTYPE, FUNC) \
  NAME##_registry::registerImpl({::tinytorch::DeviceType::DEVICE, ::tinytorch::DType::DTYPE}, FUNC)
