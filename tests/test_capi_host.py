"""Host-only checks of the C ABI (no GPU, no kernel launch): the library loads, exports every symbol that
include/ttsdpa.h declares, lays out ttsdpa_params as the header says, validates arguments and picks routes."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from tinytorch_amd import _capi

FAKE = 0x10000  # a non-NULL, 16-byte aligned address; nothing is launched in this file


def params(*dims, **kw):
    """dims = (dtype, B, Hq, Hkv, L, S, D); kw overrides struct fields afterwards."""
    p = _capi.make_params(*dims)
    p.q = p.k = p.v = p.out = FAKE
    for k, v in kw.items():
        if isinstance(v, tuple):
            for i, x in enumerate(v):
                getattr(p, k)[i] = x
        else:
            setattr(p, k, v)
    return p


def test_exports_match_header():
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in ("ttsdpa.h", "ttfused.h", "ttlinear.h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(tt(?:sdpa|fused|linear)_[a-z_]+)\s*\(", text)))
    assert declared == sorted(_capi.EXPORTS)
    L = _capi.lib()
    for name in declared:
        assert getattr(L, name) is not None
    header_version = int(re.search(r"#define\s+TTSDPA_ABI_VERSION\s+(\d+)", open(os.path.join(ROOT, "include", "ttsdpa.h")).read()).group(1))
    assert L.ttsdpa_abi_version() == header_version


def test_struct_layout_matches_header():
    # 4+4, 4 pointers, 6 ints, 12 int64, float, 2 ints, (pad), pointer, 4 int64, pointer, pointer, 2 ints
    assert ctypes.sizeof(_capi.Params) == 8 + 32 + 24 + 96 + 12 + 4 + 8 + 32 + 8 + 8 + 8
    p = _capi.make_params(_capi.BF16, 2, 32, 8, 4096, 4096, 128)
    assert p.struct_size == ctypes.sizeof(_capi.Params)
    assert list(p.q_stride) == [32 * 4096 * 128, 4096 * 128, 128]
    assert list(p.k_stride) == [8 * 4096 * 128, 4096 * 128, 128]
    assert abs(p.scale - 128 ** -0.5) < 1e-8 and p.causal == 0 and p.mask_kind == 0
    assert list(p.mask_stride) == [0, 0, 4096, 1]  # a dense [L,S] mask shared by every batch and head
    assert p.kv_len is None
    # 4+4, 4 pointers, 6 ints, 12 int64, pointer, pointer, 2 ints
    assert ctypes.sizeof(_capi.KvAppendParams) == 8 + 32 + 24 + 96 + 8 + 8 + 8
    kp = _capi.KvAppendParams()
    _capi.lib().ttsdpa_kv_append_params_init(ctypes.byref(kp), _capi.BF16, 4, 8, 1024, 2, 128)
    assert kp.struct_size == ctypes.sizeof(_capi.KvAppendParams)
    assert list(kp.kc_stride) == [8 * 1024 * 128, 1024 * 128, 128] and list(kp.vn_stride) == [8 * 2 * 128, 2 * 128, 128]


@pytest.mark.parametrize("args,route", [
    ((_capi.F32, 1, 4, 4, 128, 128, 64), _capi.ROUTE_PREFILL),       # config 1: fp32 MFMA kernel
    ((_capi.F32, 2, 8, 2, 300, 300, 128), _capi.ROUTE_PREFILL),
    ((_capi.F32, 2, 8, 2, 300, 300, 96), _capi.ROUTE_PREFILL),       # fp32 MFMA kernel: multiples of 4 up to 128 (zero columns up to 64 / 128)
    ((_capi.F32, 2, 8, 2, 300, 300, 90), _capi.ROUTE_GENERAL),
    ((_capi.F32, 2, 8, 2, 300, 300, 132), _capi.ROUTE_GENERAL),
    ((_capi.F16, 4, 32, 32, 2048, 2048, 128), _capi.ROUTE_PREFILL),  # config 2
    ((_capi.BF16, 2, 32, 8, 4096, 4096, 128), _capi.ROUTE_PREFILL),  # config 3
    ((_capi.BF16, 64, 32, 8, 1, 8192, 128), _capi.ROUTE_DECODE),     # config 4
    ((_capi.BF16, 1, 28, 4, 16384, 16384, 128), _capi.ROUTE_PREFILL),  # config 5
    ((_capi.BF16, 1, 28, 4, 1, 4096, 128), _capi.ROUTE_DECODE),      # 7 heads per KV head
    ((_capi.BF16, 4, 32, 8, 1, 4096, 96), _capi.ROUTE_DECODE),       # a multiple of 8 below 128: the head_dim-128 kernel, zero columns
    ((_capi.F16, 4, 32, 8, 1, 4096, 40), _capi.ROUTE_DECODE),
    ((_capi.BF16, 4, 32, 8, 1, 4096, 100), _capi.ROUTE_GENERAL),     # rows that are not whole 16-byte chunks
    ((_capi.BF16, 1, 8, 8, 300, 300, 64), _capi.ROUTE_PREFILL),
    ((_capi.BF16, 1, 8, 8, 300, 300, 96), _capi.ROUTE_PREFILL),
    ((_capi.F16, 1, 8, 8, 300, 300, 256), _capi.ROUTE_PREFILL),
    ((_capi.BF16, 1, 8, 8, 300, 300, 80), _capi.ROUTE_PREFILL),      # a multiple of 8: the head_dim-96 kernel with zero columns
    ((_capi.F16, 1, 8, 8, 300, 300, 8), _capi.ROUTE_PREFILL),
    ((_capi.F16, 1, 8, 8, 300, 300, 248), _capi.ROUTE_PREFILL),
    ((_capi.BF16, 1, 8, 8, 300, 300, 84), _capi.ROUTE_GENERAL),      # rows that are not whole 16-byte chunks
    ((_capi.BF16, 1, 8, 8, 300, 300, 20), _capi.ROUTE_GENERAL),
    ((_capi.BF16, 1, 64, 2, 1, 4096, 128), _capi.ROUTE_PREFILL),     # 32 rows per KV head: too many for decode
    ((_capi.BF16, 1, 8, 8, 0, 16, 128), _capi.ROUTE_NONE),
    ((_capi.BF16, 0, 8, 8, 4, 16, 128), _capi.ROUTE_NONE),
    ((_capi.BF16, 1, 8, 8, 4, 0, 128), _capi.ROUTE_ZERO),
])
def test_routes(args, route):
    rc, r = _capi.plan(params(*args))
    assert rc == 0, _capi.status_string(rc)
    assert r == route, _capi.ROUTE_NAMES[r]


def test_routes_depend_on_flags():
    base = (_capi.BF16, 2, 8, 2, 512, 512, 128)
    assert _capi.plan(params(*base, causal=1))[1] == _capi.ROUTE_PREFILL
    # an attnMask is taken by every MFMA prefill kernel; head sizes they do not cover go to the general kernel
    assert _capi.plan(params(*base, mask_kind=_capi.MASK_BOOL, mask=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 8, 2, 64, 512, 128, mask_kind=_capi.MASK_ADD, mask=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 8, 2, 512, 512, 64, mask_kind=_capi.MASK_BOOL, mask=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 8, 2, 512, 512, 80, mask_kind=_capi.MASK_BOOL, mask=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 8, 2, 512, 512, 84, mask_kind=_capi.MASK_BOOL, mask=FAKE))[1] == _capi.ROUTE_GENERAL
    assert _capi.plan(params(*base, scale=-1.0))[1] == _capi.ROUTE_GENERAL
    p = params(*base)
    p.k_stride[2] = 132  # rows not 16-byte aligned
    assert _capi.plan(p)[1] == _capi.ROUTE_GENERAL
    p = params(*base)
    p.q = FAKE + 2
    assert _capi.plan(p)[1] == _capi.ROUTE_GENERAL
    # fp32: the MFMA kernel takes attnMask and per-batch key counts, and needs 16-byte aligned rows
    f32 = (_capi.F32, 2, 8, 2, 512, 512, 128)
    assert _capi.plan(params(*f32, causal=1))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(*f32, mask_kind=_capi.MASK_ADD, mask=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(*f32, kv_len=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.F32, 2, 8, 2, 512, 512, 96, mask_kind=_capi.MASK_BOOL, mask=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.F32, 2, 8, 2, 512, 512, 98, mask_kind=_capi.MASK_BOOL, mask=FAKE))[1] == _capi.ROUTE_GENERAL
    p = params(*f32)
    p.v_stride[2] = 130
    assert _capi.plan(p)[1] == _capi.ROUTE_GENERAL
    # bottom-right aligned causal: a few new rows against a long cache stream it; one new row hides nothing
    assert _capi.plan(params(_capi.BF16, 4, 8, 2, 2, 1024, 128, causal=2))[1] == _capi.ROUTE_DECODE   # 8 rows per KV head
    assert _capi.plan(params(_capi.BF16, 4, 8, 2, 4, 1024, 128, causal=2))[1] == _capi.ROUTE_PREFILL  # 16: packed heads on the MFMA kernel
    strided = params(_capi.BF16, 4, 8, 2, 4, 1024, 128, causal=2)
    strided.q_stride[1] = 4 * 128 + 128   # heads not dense: cannot be packed, the streaming kernel takes its 16 rows
    assert _capi.plan(strided)[1] == _capi.ROUTE_DECODE
    assert _capi.plan(params(_capi.BF16, 4, 8, 2, 1, 1024, 128, causal=2))[1] == _capi.ROUTE_DECODE
    assert _capi.plan(params(_capi.BF16, 4, 8, 2, 512, 1024, 128, causal=2))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.F32, 4, 8, 2, 512, 1024, 128, causal=2))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 4, 8, 2, 2, 1024, 128, causal=2, kv_len=FAKE))[1] == _capi.ROUTE_DECODE
    # decode with causal set is the top-left triangle (only key 0 visible): not the streaming kernel's case
    assert _capi.plan(params(_capi.BF16, 4, 8, 2, 1, 1024, 128, causal=1))[1] == _capi.ROUTE_PREFILL


@pytest.mark.parametrize("mutate,status", [
    (dict(struct_size=8), _capi.ERR_ABI),
    (dict(dtype=3), _capi.ERR_DTYPE),
    (dict(q=0), _capi.ERR_NULL),
    (dict(out=0), _capi.ERR_NULL),
    (dict(Hkv=3), _capi.ERR_SHAPE),
    (dict(D=0), _capi.ERR_SHAPE),
    (dict(D=512), _capi.ERR_SHAPE),
    (dict(L=-1), _capi.ERR_SHAPE),
    (dict(mask_kind=7), _capi.ERR_MASK),
    (dict(causal=3), _capi.ERR_MASK),                                        # not a causal mode
    (dict(causal=-1), _capi.ERR_MASK),
    (dict(mask_kind=_capi.MASK_BOOL, mask=FAKE, causal=2), _capi.ERR_MASK),
    (dict(mask_kind=_capi.MASK_BOOL), _capi.ERR_NULL),                      # mask kind without a mask
    (dict(mask_kind=_capi.MASK_BOOL, mask=FAKE, causal=1), _capi.ERR_MASK),  # reference asserts on this
    (dict(mask_kind=_capi.MASK_BOOL, mask=FAKE, mask_stride=(0, 0, -64, 1)), _capi.ERR_STRIDE),
    (dict(mask_kind=_capi.MASK_ADD, mask=FAKE + 1), _capi.ERR_STRIDE),       # additive mask not element-aligned
])
def test_validation_errors(mutate, status):
    p = params(_capi.BF16, 2, 8, 2, 64, 64, 128, **mutate)
    L = _capi.lib()
    assert _capi.plan(p)[0] == status
    # every launching entry point refuses the same way, before touching the GPU
    assert L.ttsdpa_forward(ctypes.byref(p), None, 0, None) == status
    assert L.ttsdpa_general(ctypes.byref(p), None) == status
    assert L.ttsdpa_prefill(ctypes.byref(p), None) == status
    assert L.ttsdpa_decode(ctypes.byref(p), None, 0, None) == status
    assert _capi.status_string(status) not in ("ok", "unknown status")


def test_kv_len_routes_and_append_validation():
    # per-batch key counts: decode kernel, pipelined head_dim-128 prefill kernel, general kernel for the rest
    base = (_capi.BF16, 2, 32, 8, 4096, 4096, 128)
    assert _capi.plan(params(*base, causal=1))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(*base, causal=1, kv_len=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 32, 8, 4096, 4096, 64, kv_len=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 32, 8, 100, 4096, 128, kv_len=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 32, 8, 100, 4096, 80, kv_len=FAKE))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.BF16, 2, 32, 8, 100, 4096, 84, kv_len=FAKE))[1] == _capi.ROUTE_GENERAL
    assert _capi.plan(params(_capi.BF16, 8, 32, 8, 1, 4096, 128, kv_len=FAKE))[1] == _capi.ROUTE_DECODE
    assert _capi.plan(params(_capi.BF16, 8, 32, 8, 1, 4096, 128, kv_len=FAKE + 2))[0] == _capi.ERR_STRIDE
    L = _capi.lib()
    kp = _capi.KvAppendParams()
    L.ttsdpa_kv_append_params_init(ctypes.byref(kp), _capi.BF16, 4, 8, 1024, 2, 128)
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_NULL  # pointers missing
    kp.k_cache = kp.v_cache = kp.k_new = kp.v_new = FAKE
    kp.struct_size = 12
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_ABI
    kp.struct_size = ctypes.sizeof(_capi.KvAppendParams)
    kp.dtype = 9
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_DTYPE
    kp.dtype = _capi.BF16
    kp.kn_stride[2] = 64  # rows of the new tokens overlap
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_STRIDE
    kp.kn_stride[2] = 128
    kp.positions = FAKE + 1
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_STRIDE
    kp.positions = None
    kp.Lnew = 0  # nothing to append: accepted without touching the GPU
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == 0


def test_product_library_holds_no_bench_probes():
    # the measurement probes are bench tooling with a shared object of their own (bench_probes/)
    L = _capi.lib()
    assert not hasattr(L, "ttsdpa_probe") and not hasattr(L, "ttbench_probe")
    with open(os.path.join(ROOT, "include", "ttsdpa.h")) as f:
        assert "probe" not in f.read()


def test_kernel_domains_and_workspace():
    L = _capi.lib()
    fp32 = params(_capi.F32, 1, 4, 4, 128, 128, 90)  # the fp32 MFMA kernel covers the multiples of 4 up to 128
    assert L.ttsdpa_prefill(ctypes.byref(fp32), None) == _capi.ERR_UNSUPPORTED
    assert L.ttsdpa_decode(ctypes.byref(fp32), None, 0, None) == _capi.ERR_UNSUPPORTED
    # config 4 has 512 (batch, kv head) pairs: enough workgroups without splitting the cache, hence no scratch
    assert L.ttsdpa_workspace_bytes(ctypes.byref(params(_capi.BF16, 64, 32, 8, 1, 8192, 128))) == 0
    dec = params(_capi.BF16, 2, 32, 8, 1, 8192, 128)  # few pairs: the cache is split and partials need scratch
    need = L.ttsdpa_workspace_bytes(ctypes.byref(dec))
    assert need > 0 and need % 4 == 0
    assert L.ttsdpa_decode(ctypes.byref(dec), None, 0, None) == _capi.ERR_WORKSPACE
    assert L.ttsdpa_decode(ctypes.byref(dec), FAKE, need - 1, None) == _capi.ERR_WORKSPACE
    assert L.ttsdpa_forward(ctypes.byref(dec), FAKE, need - 1, None) == _capi.ERR_WORKSPACE
    # a head size between the decode kernel's: the records have the pitch of the kernel that runs (head_dim 128 here)
    assert L.ttsdpa_workspace_bytes(ctypes.byref(params(_capi.BF16, 2, 32, 8, 1, 8192, 96))) == need
    assert L.ttsdpa_workspace_bytes(ctypes.byref(params(_capi.BF16, 2, 32, 8, 1, 8192, 40))) == \
        L.ttsdpa_workspace_bytes(ctypes.byref(params(_capi.BF16, 2, 32, 8, 1, 8192, 64)))
    short = params(_capi.BF16, 2, 8, 2, 1, 64, 128)
    assert L.ttsdpa_workspace_bytes(ctypes.byref(short)) == 0          # one split: no scratch
    assert L.ttsdpa_workspace_bytes(ctypes.byref(fp32)) == 0
    big = params(_capi.BF16, 1, 64, 2, 1, 4096, 128)
    assert L.ttsdpa_decode(ctypes.byref(big), None, 0, None) == _capi.ERR_UNSUPPORTED


def test_host_wrapper_argument_errors():
    import torch
    from tinytorch_amd import sdpAttention
    q = torch.zeros(1, 2, 4, 8)
    with pytest.raises(RuntimeError, match="GPU only"):   # no CPU fallback behind this package
        sdpAttention(q, q, q)
    with pytest.raises(NotImplementedError):
        sdpAttention(q, q, q, dropoutP=0.1)
    with pytest.raises(ValueError):
        sdpAttention(q[0], q[0], q[0])


def test_fused_ops_argument_checks_without_a_gpu():
    """include/ttfused.h: empty problems return before any launch; bad arguments are refused the same way."""
    L = _capi.lib()
    assert L.ttfused_rms_norm(_capi.BF16, None, None, None, 0, 4096, 1e-6, None) == 0
    assert L.ttfused_rms_norm(_capi.BF16, FAKE, None, None, 4, 4096, 1e-6, None) == _capi.ERR_NULL
    assert L.ttfused_rms_norm(9, FAKE, None, FAKE, 4, 4096, 1e-6, None) == _capi.ERR_DTYPE
    assert L.ttfused_rms_norm(_capi.F32, FAKE, None, FAKE, -4, 4096, 1e-6, None) == _capi.ERR_SHAPE
    assert L.ttfused_rms_norm(_capi.F32, FAKE, None, FAKE, 4, 1 << 31, 1e-6, None) == _capi.ERR_SHAPE
    assert L.ttfused_add_rms_norm(_capi.F16, FAKE, FAKE, None, 4, 128, 1e-6, None) == _capi.ERR_NULL   # weight is required
    assert L.ttfused_add_rms_norm(_capi.F16, FAKE, FAKE, FAKE, 0, 128, 1e-6, None) == 0
    assert L.ttfused_silu_mul(_capi.F32, FAKE, None, 4, 128, None) == _capi.ERR_NULL
    assert L.ttfused_silu_mul(_capi.F32, None, None, 4, 0, None) == 0
    assert L.ttfused_softmax(_capi.F32, FAKE, FAKE, 4, 8, -1, 0, None) == _capi.ERR_SHAPE
    assert L.ttfused_softmax(_capi.F32, None, None, 4, 0, 1, 1, None) == 0


def test_paged_cache_routes_and_validation():
    """block_table: decode kernel for pages of 32 rows or more, MFMA prefill kernels for 64 or more, general kernel
    otherwise; page sizes are powers of two."""
    dec = (_capi.BF16, 4, 32, 8, 1, 4096, 128)
    paged = dict(block_table=FAKE, page_size=64, block_table_stride=64)
    assert _capi.plan(params(*dec, **paged))[1] == _capi.ROUTE_DECODE
    assert _capi.plan(params(*dec, **paged, kv_len=FAKE))[1] == _capi.ROUTE_DECODE
    assert _capi.plan(params(*dec, block_table=FAKE, page_size=16, block_table_stride=256))[1] == _capi.ROUTE_GENERAL
    # the MFMA prefill kernels stage 64-key tiles: pages of 64 rows or more
    assert _capi.plan(params(_capi.BF16, 4, 32, 8, 512, 4096, 128, causal=2, **paged))[1] == _capi.ROUTE_PREFILL
    assert _capi.plan(params(_capi.F32, 4, 32, 8, 1, 4096, 128, **paged))[1] == _capi.ROUTE_PREFILL
    small = dict(block_table=FAKE, page_size=32, block_table_stride=128)
    assert _capi.plan(params(_capi.BF16, 4, 32, 8, 512, 4096, 128, causal=2, **small))[1] == _capi.ROUTE_GENERAL
    assert _capi.plan(params(_capi.F32, 4, 32, 8, 1, 4096, 128, **small))[1] == _capi.ROUTE_GENERAL
    assert _capi.plan(params(*dec, **small))[1] == _capi.ROUTE_DECODE
    assert _capi.plan(params(*dec, block_table=FAKE, page_size=48, block_table_stride=128))[0] == _capi.ERR_SHAPE
    assert _capi.plan(params(*dec, block_table=FAKE, page_size=0, block_table_stride=128))[0] == _capi.ERR_SHAPE
    assert _capi.plan(params(*dec, block_table=FAKE + 2, page_size=64, block_table_stride=64))[0] == _capi.ERR_STRIDE
    assert _capi.plan(params(*dec, block_table=FAKE, page_size=64, block_table_stride=8))[0] == _capi.ERR_STRIDE  # rows of the table overlap
    L = _capi.lib()
    kp = _capi.KvAppendParams()
    L.ttsdpa_kv_append_params_init(ctypes.byref(kp), _capi.BF16, 4, 8, 4096, 1, 128)
    kp.k_cache = kp.v_cache = kp.k_new = kp.v_new = FAKE
    kp.block_table, kp.page_size, kp.block_table_stride = FAKE, 24, 64
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_SHAPE
    kp.block_table, kp.page_size = FAKE + 1, 64
    assert L.ttsdpa_kv_append(ctypes.byref(kp), None) == _capi.ERR_STRIDE


def test_linear_routes_and_validation():
    L = _capi.lib()
    r = ctypes.c_int(-1)

    def plan(dtype, M, N, K, ldx=None, ldw=None, ldo=None, x=FAKE, w=FAKE, out=FAKE):
        rc = L.ttlinear_plan(dtype, x, w, None, out, M, N, K, ldx or K, ldw or K, ldo or N, ctypes.byref(r))
        return rc, _capi.LINEAR_ROUTE_NAMES.get(r.value)

    assert plan(_capi.BF16, 8192, 4096, 4096) == (0, "mfma")
    assert plan(_capi.F16, 100, 12, 64) == (0, "mfma")
    assert plan(_capi.F32, 8192, 4096, 4096) == (0, "mfma")          # fp32 on the fp32 matrix cores
    assert plan(_capi.F32, 8192, 4096, 4000) == (0, "mfma")          # K a multiple of 32 suffices in fp32
    assert plan(_capi.F32, 8192, 4096, 4008) == (0, "general")
    assert plan(_capi.BF16, 8192, 4096, 4000) == (0, "general")      # K not a multiple of 64
    assert plan(_capi.BF16, 8192, 4095, 4096) == (0, "general")      # N not a multiple of 4
    assert plan(_capi.BF16, 64, 64, 64, x=FAKE + 2) == (0, "general")  # rows not 16-byte aligned
    assert plan(_capi.BF16, 0, 64, 64) == (0, "none")
    assert plan(_capi.BF16, 64, 64, 0) == (0, "general")             # K == 0: the bias
    assert plan(7, 64, 64, 64)[0] == _capi.ERR_DTYPE
    assert plan(_capi.BF16, -1, 64, 64)[0] == _capi.ERR_SHAPE
    assert plan(_capi.BF16, 64, 64, 64, ldx=32)[0] == _capi.ERR_STRIDE
    assert plan(_capi.BF16, 64, 64, 64, x=None)[0] == _capi.ERR_NULL
    assert L.ttlinear_forward(_capi.BF16, None, None, None, None, 0, 64, 64, 64, 64, 64, None) == 0
    assert L.ttlinear_forward(_capi.BF16, FAKE, FAKE, None, None, 8, 64, 64, 64, 64, 64, None) == _capi.ERR_NULL


def test_backward_params_layout_routes_and_validation():
    """struct ttsdpa_backward_params as the header lays it out; plan and validation of ttsdpa_backward without a GPU."""
    L = _capi.lib()
    bp = _capi.BackwardParams()
    L.ttsdpa_backward_params_init(ctypes.byref(bp), _capi.BF16, 2, 8, 2, 64, 96, 128)
    assert bp.struct_size == ctypes.sizeof(_capi.BackwardParams) == 8 + ctypes.sizeof(_capi.Params) + 4 * 8 + 4 * 24
    assert bp.fwd.struct_size == ctypes.sizeof(_capi.Params) and bp.fwd.L == 64 and bp.fwd.S == 96
    assert list(bp.dq_stride) == list(bp.fwd.q_stride) == [8 * 64 * 128, 64 * 128, 128]
    assert list(bp.dk_stride) == list(bp.dv_stride) == list(bp.fwd.k_stride) == [2 * 96 * 128, 96 * 128, 128]
    r = ctypes.c_int(-1)
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == _capi.ERR_NULL      # no tensors yet
    bp.fwd.q = bp.fwd.k = bp.fwd.v = bp.fwd.out = FAKE
    bp.dout = bp.dq = bp.dk = bp.dv = FAKE
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value in (_capi.ROUTE_GENERAL, _capi.ROUTE_PREFILL)
    assert L.ttsdpa_backward_workspace_bytes(ctypes.byref(bp)) >= 2 * 8 * 64 * 2 * 4
    assert L.ttsdpa_backward(ctypes.byref(bp), None, 0, None) == _capi.ERR_WORKSPACE
    bp.dk = None
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == _capi.ERR_NULL
    bp.dk = FAKE + 1
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == _capi.ERR_STRIDE
    bp.dk = FAKE
    bp.dv_stride[2] = 64
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == _capi.ERR_STRIDE
    bp.dv_stride[2] = 128
    bp.fwd.block_table, bp.fwd.page_size, bp.fwd.block_table_stride = FAKE, 64, 64
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == _capi.ERR_UNSUPPORTED
    bp.fwd.block_table = None
    bp.struct_size -= 8
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == _capi.ERR_ABI
    # fp32: the fp32 matrix-core pair at head_dim 64 / 128 with 16-byte aligned rows, else the vector-ALU kernels
    L.ttsdpa_backward_params_init(ctypes.byref(bp), _capi.F32, 1, 4, 4, 32, 32, 64)
    bp.fwd.q = bp.fwd.k = bp.fwd.v = bp.fwd.out = bp.dout = bp.dq = bp.dk = bp.dv = FAKE
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value == _capi.ROUTE_PREFILL
    bp.dq_stride[2] = 66
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value == _capi.ROUTE_GENERAL
    bp.dq_stride[2] = 64
    bp.fwd.k = FAKE + 4
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value == _capi.ROUTE_GENERAL
    # other head sizes: multiples of 4 up to 128 on the same pair (zero columns up to 64 / 128), the rest on the vector ALUs
    for D, route in ((96, _capi.ROUTE_PREFILL), (20, _capi.ROUTE_PREFILL), (90, _capi.ROUTE_GENERAL), (160, _capi.ROUTE_GENERAL)):
        L.ttsdpa_backward_params_init(ctypes.byref(bp), _capi.F32, 1, 4, 4, 32, 32, D)
        bp.fwd.q = bp.fwd.k = bp.fwd.v = bp.fwd.out = bp.dout = bp.dq = bp.dk = bp.dv = FAKE
        assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value == route, D
    # 16-bit tensors: multiples of 8 up to 128
    for D, route in ((80, _capi.ROUTE_PREFILL), (8, _capi.ROUTE_PREFILL), (84, _capi.ROUTE_GENERAL), (136, _capi.ROUTE_GENERAL)):
        L.ttsdpa_backward_params_init(ctypes.byref(bp), _capi.BF16, 1, 4, 4, 32, 32, D)
        bp.fwd.q = bp.fwd.k = bp.fwd.v = bp.fwd.out = bp.dout = bp.dq = bp.dk = bp.dv = FAKE
        assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value == route, D
    L.ttsdpa_backward_params_init(ctypes.byref(bp), _capi.F32, 0, 4, 4, 32, 32, 64)
    assert L.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0 and r.value == _capi.ROUTE_NONE


def test_build_params_refuses_a_mask_on_another_device():
    """The mask's address goes to the kernels as it is: a mask that does not live with the tensors must be refused on
    the host (a host pointer dereferenced by a kernel is a GPU memory fault)."""
    import torch
    import tinytorch_amd

    q = torch.zeros(1, 2, 4, 8)
    k = torch.zeros(1, 2, 6, 8)
    out = torch.empty_like(q)
    mask = torch.ones(4, 6, dtype=torch.bool, device="meta")
    with pytest.raises(RuntimeError, match="attnMask must live on the device"):
        tinytorch_amd.build_params(q, k, k, out, False, mask)
    p = tinytorch_amd.build_params(q, k, k, out, False, torch.ones(4, 6, dtype=torch.bool))  # same device: accepted
    assert p.mask_kind == 1


def test_static_scratch_decode_refuses_what_does_not_fit():
    """ttsdpa_decode_static holds TTSDPA_STATIC_SCRATCH_BYTES of split-KV records: a call that needs more is refused
    before anything is launched or looked up (so this needs no GPU), with a status of its own."""
    lib = _capi.lib()
    header = open(os.path.join(ROOT, "include", "ttsdpa.h")).read()
    assert "#define TTSDPA_STATIC_SCRATCH_BYTES (2u << 20)" in header and _capi.STATIC_SCRATCH_BYTES == 2 << 20
    # 16 rows per KV head against a very long cache, few (batch, head) pairs: 64 splits of 16 x 130 floats per pair
    p = _capi.make_params(_capi.BF16, 4, 64, 4, 1, 1 << 20, 128)
    p.q = p.k = p.v = p.out = 0x1000  # never dereferenced
    need = lib.ttsdpa_workspace_bytes(ctypes.byref(p))
    assert need > _capi.STATIC_SCRATCH_BYTES
    assert lib.ttsdpa_decode_static(ctypes.byref(p), None) == _capi.ERR_STATIC_SCRATCH
    assert "static" in _capi.status_string(_capi.ERR_STATIC_SCRATCH)
    # outside the decode kernel's domain: the same answer as ttsdpa_decode
    fp32 = _capi.make_params(_capi.F32, 1, 4, 4, 1, 1024, 128)
    fp32.q = fp32.k = fp32.v = fp32.out = 0x1000
    assert lib.ttsdpa_decode_static(ctypes.byref(fp32), None) == _capi.ERR_UNSUPPORTED
    assert lib.ttsdpa_decode_static(None, None) == _capi.ERR_NULL
