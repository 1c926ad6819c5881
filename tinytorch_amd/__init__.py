"""MI355X-native scaled-dot-product attention behind TinyTorch's ``function::sdpAttention`` interface.

The compute path is the HIP library ``tinytorch_amd/lib/libttsdpa.so`` (C ABI: include/ttsdpa.h).  Importing this
package loads it and fails if it has not been built.
"""
from . import _capi

_capi.lib()  # fail loudly when the extension is missing

from .function import sdpAttention, kvCacheAppend, build_params  # noqa: E402

__all__ = ["sdpAttention", "kvCacheAppend", "build_params"]
