"""ctypes binding of the C ABI declared in include/ttsdpa.h (tinytorch_amd/lib/libttsdpa.so).

The library is the product: when it is missing the import fails loudly — there is no other compute path.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libttsdpa.so")

F32, F16, BF16 = 0, 1, 2
MASK_NONE, MASK_BOOL, MASK_ADD = 0, 1, 2
CAUSAL_NONE, CAUSAL_TOP_LEFT, CAUSAL_BOTTOM_RIGHT = 0, 1, 2
ROUTE_NONE, ROUTE_GENERAL, ROUTE_PREFILL, ROUTE_DECODE, ROUTE_ZERO = 0, 1, 2, 3, 4
ROUTE_NAMES = {0: "none", 1: "general", 2: "prefill", 3: "decode", 4: "zero"}

OK = 0
ERR_NULL, ERR_DTYPE, ERR_SHAPE, ERR_STRIDE, ERR_MASK, ERR_WORKSPACE, ERR_UNSUPPORTED, ERR_ABI, ERR_STATIC_SCRATCH = range(-1, -10, -1)
STATIC_SCRATCH_BYTES = 2 << 20

EXPORTS = [
    "ttsdpa_abi_version", "ttsdpa_status_string", "ttsdpa_params_init", "ttsdpa_plan", "ttsdpa_workspace_bytes",
    "ttsdpa_forward", "ttsdpa_prefill", "ttsdpa_decode", "ttsdpa_decode_static", "ttsdpa_general",
    "ttsdpa_kv_append_params_init", "ttsdpa_kv_append",
    "ttsdpa_backward_params_init", "ttsdpa_backward_plan", "ttsdpa_backward_workspace_bytes", "ttsdpa_backward",
    # include/ttfused.h
    "ttfused_rms_norm", "ttfused_add_rms_norm", "ttfused_silu_mul", "ttfused_softmax", "ttfused_softmax_backward",
    # include/ttlinear.h
    "ttlinear_forward", "ttlinear_plan", "ttlinear_matmul", "ttlinear_matmul_batched", "ttlinear_matmul_workspace_bytes",
]
LINEAR_ROUTE_NAMES = {0: "none", 1: "mfma", 2: "general"}


class Params(ctypes.Structure):
    """struct ttsdpa_params"""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("Hkv", ctypes.c_int32),
        ("L", ctypes.c_int32), ("S", ctypes.c_int32), ("D", ctypes.c_int32),
        ("q_stride", ctypes.c_int64 * 3),
        ("k_stride", ctypes.c_int64 * 3),
        ("v_stride", ctypes.c_int64 * 3),
        ("o_stride", ctypes.c_int64 * 3),
        ("scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("mask_kind", ctypes.c_int32),
        ("mask", ctypes.c_void_p),
        ("mask_stride", ctypes.c_int64 * 4),
        ("kv_len", ctypes.c_void_p),
        ("block_table", ctypes.c_void_p),
        ("page_size", ctypes.c_int32),
        ("block_table_stride", ctypes.c_int32),
    ]


class BackwardParams(ctypes.Structure):
    """struct ttsdpa_backward_params"""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("reserved", ctypes.c_uint32),
        ("fwd", Params),
        ("dout", ctypes.c_void_p),
        ("dq", ctypes.c_void_p),
        ("dk", ctypes.c_void_p),
        ("dv", ctypes.c_void_p),
        ("dout_stride", ctypes.c_int64 * 3),
        ("dq_stride", ctypes.c_int64 * 3),
        ("dk_stride", ctypes.c_int64 * 3),
        ("dv_stride", ctypes.c_int64 * 3),
    ]


class KvAppendParams(ctypes.Structure):
    """struct ttsdpa_kv_append_params"""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("k_cache", ctypes.c_void_p),
        ("v_cache", ctypes.c_void_p),
        ("k_new", ctypes.c_void_p),
        ("v_new", ctypes.c_void_p),
        ("B", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("Smax", ctypes.c_int32),
        ("Lnew", ctypes.c_int32), ("D", ctypes.c_int32),
        ("position", ctypes.c_int32),
        ("kc_stride", ctypes.c_int64 * 3),
        ("vc_stride", ctypes.c_int64 * 3),
        ("kn_stride", ctypes.c_int64 * 3),
        ("vn_stride", ctypes.c_int64 * 3),
        ("positions", ctypes.c_void_p),
        ("block_table", ctypes.c_void_p),
        ("page_size", ctypes.c_int32),
        ("block_table_stride", ctypes.c_int32),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "tinytorch_amd: %s is missing — build it with `make -C tinytorch_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback path" % LIB_PATH)
        # torch ships its own HIP runtime (same SONAME as the system one).  Device pointers and streams handed to the
        # library come from torch, so the library must bind to that copy: load torch's first.
        import torch  # noqa: F401
        L = ctypes.CDLL(LIB_PATH)
        P = ctypes.POINTER(Params)
        L.ttsdpa_abi_version.restype = ctypes.c_int
        L.ttsdpa_status_string.argtypes = [ctypes.c_int]
        L.ttsdpa_status_string.restype = ctypes.c_char_p
        L.ttsdpa_params_init.argtypes = [P] + [ctypes.c_int] * 7
        L.ttsdpa_params_init.restype = None
        L.ttsdpa_plan.argtypes = [P, ctypes.POINTER(ctypes.c_int)]
        L.ttsdpa_plan.restype = ctypes.c_int
        L.ttsdpa_workspace_bytes.argtypes = [P]
        L.ttsdpa_workspace_bytes.restype = ctypes.c_size_t
        L.ttsdpa_forward.argtypes = [P, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.ttsdpa_forward.restype = ctypes.c_int
        L.ttsdpa_prefill.argtypes = [P, ctypes.c_void_p]
        L.ttsdpa_prefill.restype = ctypes.c_int
        L.ttsdpa_decode.argtypes = [P, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.ttsdpa_decode.restype = ctypes.c_int
        L.ttsdpa_decode_static.argtypes = [P, ctypes.c_void_p]
        L.ttsdpa_decode_static.restype = ctypes.c_int
        L.ttsdpa_general.argtypes = [P, ctypes.c_void_p]
        L.ttsdpa_general.restype = ctypes.c_int
        L.ttsdpa_kv_append_params_init.argtypes = [ctypes.POINTER(KvAppendParams)] + [ctypes.c_int] * 6
        L.ttsdpa_kv_append_params_init.restype = None
        L.ttsdpa_kv_append.argtypes = [ctypes.POINTER(KvAppendParams), ctypes.c_void_p]
        L.ttsdpa_kv_append.restype = ctypes.c_int
        BP = ctypes.POINTER(BackwardParams)
        L.ttsdpa_backward_params_init.argtypes = [BP] + [ctypes.c_int] * 7
        L.ttsdpa_backward_params_init.restype = None
        L.ttsdpa_backward_plan.argtypes = [BP, ctypes.POINTER(ctypes.c_int)]
        L.ttsdpa_backward_plan.restype = ctypes.c_int
        L.ttsdpa_backward_workspace_bytes.argtypes = [BP]
        L.ttsdpa_backward_workspace_bytes.restype = ctypes.c_size_t
        L.ttsdpa_backward.argtypes = [BP, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.ttsdpa_backward.restype = ctypes.c_int
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        L.ttfused_rms_norm.argtypes = [ctypes.c_int, vp, vp, vp, i64, i64, ctypes.c_float, vp]
        L.ttfused_rms_norm.restype = ctypes.c_int
        L.ttfused_add_rms_norm.argtypes = [ctypes.c_int, vp, vp, vp, i64, i64, ctypes.c_float, vp]
        L.ttfused_add_rms_norm.restype = ctypes.c_int
        L.ttfused_silu_mul.argtypes = [ctypes.c_int, vp, vp, i64, i64, vp]
        L.ttfused_silu_mul.restype = ctypes.c_int
        L.ttfused_softmax.argtypes = [ctypes.c_int, vp, vp, i64, i64, i64, ctypes.c_int, vp]
        L.ttfused_softmax.restype = ctypes.c_int
        L.ttfused_softmax_backward.argtypes = [ctypes.c_int, vp, vp, vp, i64, i64, i64, ctypes.c_int, vp]
        L.ttfused_softmax_backward.restype = ctypes.c_int
        L.ttlinear_forward.argtypes = [ctypes.c_int, vp, vp, vp, vp] + [i64] * 6 + [vp]
        L.ttlinear_forward.restype = ctypes.c_int
        L.ttlinear_plan.argtypes = [ctypes.c_int, vp, vp, vp, vp] + [i64] * 6 + [ctypes.POINTER(ctypes.c_int)]
        L.ttlinear_plan.restype = ctypes.c_int
        L.ttlinear_matmul_workspace_bytes.argtypes = [ctypes.c_int, i64, i64, i64, ctypes.c_int, ctypes.c_int]
        L.ttlinear_matmul_workspace_bytes.restype = ctypes.c_size_t
        L.ttlinear_matmul.argtypes = [ctypes.c_int, vp, vp, vp, vp, i64, i64, i64, ctypes.c_int, ctypes.c_int, i64, i64, i64,
                                      vp, ctypes.c_size_t, vp]
        L.ttlinear_matmul.restype = ctypes.c_int
        i64p = ctypes.POINTER(ctypes.c_int64)
        L.ttlinear_matmul_batched.argtypes = [ctypes.c_int, vp, vp, vp, vp, i64, i64, i64, ctypes.c_int, ctypes.c_int, i64, i64,
                                              i64, ctypes.c_int, i64p, i64p, i64p, i64, vp, ctypes.c_size_t, vp]
        L.ttlinear_matmul_batched.restype = ctypes.c_int
        if L.ttsdpa_abi_version() != 7:
            raise ImportError("tinytorch_amd: libttsdpa.so ABI version mismatch")
        _lib = L
    return _lib


def status_string(rc):
    return lib().ttsdpa_status_string(rc).decode()


def make_params(dtype, B, Hq, Hkv, L, S, D):
    p = Params()
    lib().ttsdpa_params_init(ctypes.byref(p), dtype, B, Hq, Hkv, L, S, D)
    return p


def plan(p):
    """-> (status, route)"""
    r = ctypes.c_int(-1)
    rc = lib().ttsdpa_plan(ctypes.byref(p), ctypes.byref(r))
    return rc, r.value
