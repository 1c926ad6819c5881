"""MI355X-native scaled-dot-product attention behind TinyTorch's ``function::sdpAttention`` interface, with the
row-wise ops that sit next to it in a transformer block (rmsNorm, fusedAddRmsNorm, siluMul, softmax).

The compute path is the HIP library ``tinytorch_amd/lib/libttsdpa.so`` (C ABI: include/ttsdpa.h, include/ttfused.h, include/ttlinear.h).  Importing this
package loads it and fails if it has not been built.
"""
from . import _capi

_capi.lib()  # fail loudly when the extension is missing

from .function import (sdpAttention, kvCacheAppend, build_params, rmsNorm, fusedAddRmsNorm, siluMul, softmax,  # noqa: E402
                       logSoftmax, linear, sdpAttentionBackward, build_backward_params, matmul, linearBackward, softmaxBackward,
                       logSoftmaxBackward)

__all__ = ["sdpAttention", "kvCacheAppend", "build_params", "rmsNorm", "fusedAddRmsNorm", "siluMul", "softmax",
           "logSoftmax", "linear", "sdpAttentionBackward", "build_backward_params", "matmul",
           "linearBackward", "softmaxBackward", "logSoftmaxBackward"]
