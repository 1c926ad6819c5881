// Umbrella header of the host layer (the reference's is src/TinyTorch.h): everything a caller of
// tinytorch::function::sdpAttention and of the row-wise ops next to it needs.
#pragma once

#include "Dispatch.h"
#include "FuncFused.h"
#include "FuncNNLayer.h"
#include "Function.h"
#include "Macros.h"
#include "OpAttention.h"
#include "OpFused.h"
#include "OpLinalg.h"
#include "Tensor.h"
