// op::matmul with the reference's signature (src/Operation/OpLinalg.h, implementation src/Operation/OpLinalg.cpp:244-276),
// registered for {GPU, Float32 / Float16 / BFloat16}.  The GPU implementation covers the call the linear layer makes —
// matmul(input, weight, false, true, bias), reference src/Function/FuncNNLayer.h:14-19 — through include/ttlinear.h;
// other transpose flags fail loudly (ASSERT), like every call this host layer does not serve.
#pragma once

#include "Dispatch.h"

namespace tinytorch::op {

// a [..., K], b [N, K] with transA == false, transB == true (the linear layer); bias undefined or [N].  Returns [..., N].
// The other flag pairs take 2-D operands: a [M, K] ([K, M] with transA; leading batch axes allowed without it), b [K, N]
// ([N, K] with transB).
using MatmulOpFn = Tensor (*)(const Tensor& a, const Tensor& b, bool transA, bool transB, const Tensor& bias);

DEFINE_OP(matmul, MatmulOpFn)

void registerLinalgGpu();
STATIC_CALL(registerLinalgGpu);

}  // namespace tinytorch::op
