// Umbrella header of the host layer (the reference's is src/TinyTorch.h): everything a caller of
// tinytorch::function::sdpAttention needs.
#pragma once

#include "Dispatch.h"
#include "FuncNNLayer.h"
#include "Function.h"
#include "Macros.h"
#include "OpAttention.h"
#include "Tensor.h"
