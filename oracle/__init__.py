"""TEST INFRASTRUCTURE — numpy/ctypes access to the parity checkers.  Never imported by the product package.

``sdpa_f32`` and friends call ``oracle/libsdpa_oracle.so`` (this repository's C restatement of TinyTorch's fp32 CPU
attention, reference src/Function/FuncNNLayer.h:231-266).  ``ref_*`` call ``oracle/_ref/libtt_ref.so``, the real
TinyTorch CPU library compiled by ``oracle/Makefile``, when that file is present.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libsdpa_oracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libtt_ref.so")

F32, F16, BF16 = 0, 1, 2
MASK_NONE, MASK_BOOL, MASK_FLOAT = 0, 1, 2
_DTYPES = {"f32": F32, "fp32": F32, "f16": F16, "fp16": F16, "bf16": BF16}

_c_f32p = ctypes.POINTER(ctypes.c_float)
_c_u16p = ctypes.POINTER(ctypes.c_uint16)
_c_i64p = ctypes.POINTER(ctypes.c_int64)
_i64 = ctypes.c_int64


def build(ref=True):
    """Compile the C restatement (always) and, where the reference tree is mounted, oracle/_ref."""
    subprocess.run(["make", "-C", _HERE, "oracle"], check=True)
    if ref and os.path.isdir("/root/reference/src"):
        subprocess.run(["make", "-C", _HERE, "ref", "-j8"], check=True)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build(ref=False)
        L = ctypes.CDLL(ORACLE_SO)
        L.oracle_round_array.argtypes = [_c_f32p, _c_f32p, _c_u16p, _i64, ctypes.c_int]
        L.oracle_round_array.restype = None
        L.oracle_bits_to_f32_array.argtypes = [_c_u16p, _c_f32p, _i64, ctypes.c_int]
        L.oracle_bits_to_f32_array.restype = None
        L.oracle_randn.argtypes = [ctypes.c_uint64, ctypes.c_uint64, _i64, ctypes.c_float, _c_f32p, ctypes.c_int]
        L.oracle_randn.restype = None
        L.oracle_sdpa_f32.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p] + [_i64] * 6 + [
            ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_int]
        L.oracle_sdpa_f32.restype = ctypes.c_int
        L.oracle_sdpa_rows_f32.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p] + [_i64] * 6 + [
            ctypes.c_int, ctypes.c_float, _c_i64p, _i64, ctypes.c_int]
        L.oracle_sdpa_rows_f32.restype = ctypes.c_int
        L.oracle_sdpa_backward_f32.argtypes = [_c_f32p] * 7 + [_i64] * 6 + [
            ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_int]
        L.oracle_sdpa_backward_f32.restype = ctypes.c_int
        L.oracle_rms_norm.argtypes = [_c_f32p, _c_f32p, _c_f32p, _i64, _i64, ctypes.c_float, ctypes.c_int]
        L.oracle_rms_norm.restype = None
        L.oracle_fused_add_rms_norm.argtypes = [_c_f32p, _c_f32p, _c_f32p, _i64, _i64, ctypes.c_float, ctypes.c_int]
        L.oracle_fused_add_rms_norm.restype = None
        L.oracle_silu_mul.argtypes = [_c_f32p, _c_f32p, _i64, _i64, ctypes.c_int]
        L.oracle_silu_mul.restype = None
        L.oracle_softmax.argtypes = [_c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int, ctypes.c_int]
        L.oracle_softmax.restype = None
        L.oracle_softmax_backward.argtypes = [_c_f32p, _c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int, ctypes.c_int]
        L.oracle_softmax_backward.restype = None
        L.oracle_linear.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int]
        L.oracle_linear.restype = None
        L.oracle_matmul.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.oracle_matmul.restype = None
        _lib = L
    return _lib


def have_ref():
    return os.path.exists(REF_SO)


def ref():
    global _ref
    if _ref is None:
        R = ctypes.CDLL(REF_SO)
        R.tt_ref_round_trip.argtypes = [_c_f32p, _c_f32p, _i64, ctypes.c_int]
        R.tt_ref_round_trip.restype = ctypes.c_int
        R.tt_ref_sdpa_f32.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p] + [_i64] * 6 + [
            ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
            ctypes.POINTER(ctypes.c_int64)]
        R.tt_ref_sdpa_f32.restype = ctypes.c_int
        R.tt_ref_sdpa_f32_gqa5d.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p] + [_i64] * 6 + [ctypes.c_int]
        R.tt_ref_sdpa_f32_gqa5d.restype = ctypes.c_int
        R.tt_ref_rms_norm.argtypes = [_c_f32p, _c_f32p, _c_f32p, _i64, _i64, ctypes.c_float]
        R.tt_ref_rms_norm.restype = ctypes.c_int
        R.tt_ref_fused_add_rms_norm.argtypes = [_c_f32p, _c_f32p, _c_f32p, _i64, _i64, ctypes.c_float]
        R.tt_ref_fused_add_rms_norm.restype = ctypes.c_int
        R.tt_ref_silu_mul.argtypes = [_c_f32p, _c_f32p, _i64, _i64]
        R.tt_ref_silu_mul.restype = ctypes.c_int
        R.tt_ref_softmax.argtypes = [_c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int]
        R.tt_ref_softmax.restype = ctypes.c_int
        R.tt_ref_softmax_backward.argtypes = [_c_f32p, _c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int]
        R.tt_ref_softmax_backward.restype = ctypes.c_int
        R.tt_ref_linear.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p, _i64, _i64, _i64]
        R.tt_ref_linear.restype = ctypes.c_int
        R.tt_ref_matmul.argtypes = [_c_f32p, _c_f32p, _c_f32p, _c_f32p, _i64, _i64, _i64, ctypes.c_int, ctypes.c_int]
        R.tt_ref_matmul.restype = ctypes.c_int
        _ref = R
    return _ref


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(_c_f32p)


def default_threads():
    return max(1, min(16, os.cpu_count() or 1))


def randn(seed, stream, shape, mul=1.0, nthreads=None):
    """i.i.d. N(0,1)*mul as float32; element i depends only on (seed, stream, i)."""
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n, dtype=np.float32)
    lib().oracle_randn(seed, stream, n, mul, _p(out), nthreads or default_threads())
    return out.reshape(shape)


def round_to(x, dtype):
    """Round fp32 -> dtype (RNE) -> (fp32 values of the rounded numbers, uint16 bit patterns or None)."""
    d = _DTYPES[dtype] if isinstance(dtype, str) else dtype
    x = _f32(x)
    if d == F32:
        return x.copy(), None
    vals = np.empty_like(x)
    bits = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_round_array(_p(x), _p(vals), bits.ctypes.data_as(_c_u16p), x.size, d)
    return vals, bits


def bits_to_f32(bits, dtype):
    d = _DTYPES[dtype] if isinstance(dtype, str) else dtype
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().oracle_bits_to_f32_array(bits.ctypes.data_as(_c_u16p), _p(out), bits.size, d)
    return out


def _dims(q, k, v):
    B, Hq, L, D = q.shape
    Bk, Hkv, S, Dk = k.shape
    assert v.shape == k.shape and Bk == B and Dk == D and Hq % Hkv == 0
    return B, Hq, Hkv, L, S, D


def _mask_args(mask, L, S, any_shape=False):
    if mask is None:
        return MASK_NONE, None, None
    if mask.dtype == np.bool_ or mask.dtype == np.uint8:
        m = np.ascontiguousarray(mask, dtype=np.uint8)
        kind = MASK_BOOL
    else:
        m = _f32(mask)
        kind = MASK_FLOAT
    assert any_shape or m.shape == (L, S)
    return kind, m, ctypes.c_void_p(m.ctypes.data)


def sdpa_f32(q, k, v, causal=False, scale=None, mask=None, nthreads=None):
    """The restated reference CPU path: q [B,Hq,L,D], k/v [B,Hkv,S,D] float32 -> [B,Hq,L,D] float32."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, Hq, Hkv, L, S, D = _dims(q, k, v)
    sc = np.float32(1.0) / np.sqrt(np.float32(D)) if scale is None else np.float32(scale)
    if mask is not None and tuple(mask.shape) != (L, S):
        # attnMask of another shape: the reference's bias add broadcasts it over [B,Hq,L,S] (reference
        # src/Function/FuncNNLayer.h:249-260), so every (batch, head) slice sees its own [L,S] slice of the mask.
        full = np.broadcast_to(mask, (B, Hq, L, S))
        G = Hq // Hkv
        out = np.empty(q.shape, dtype=np.float32)
        for b in range(B):
            for h in range(Hq):
                out[b, h] = sdpa_f32(q[b:b + 1, h:h + 1], k[b:b + 1, h // G:h // G + 1], v[b:b + 1, h // G:h // G + 1],
                                     scale=sc, mask=np.ascontiguousarray(full[b, h]), nthreads=nthreads)[0, 0]
        return out
    kind, keep, mp = _mask_args(mask, L, S)
    out = np.empty(q.shape, dtype=np.float32)
    rc = lib().oracle_sdpa_f32(_p(q), _p(k), _p(v), _p(out), B, Hq, Hkv, L, S, D, int(bool(causal)), float(sc), kind,
                               mp, nthreads or default_threads())
    if rc != 0:
        raise RuntimeError("oracle_sdpa_f32 failed: %d" % rc)
    return out


def sdpa_rows_f32(q, k, v, rows, causal=False, scale=None, nthreads=None):
    """Restated path for selected (b, h, l) triples only -> [len(rows), D]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, Hq, Hkv, L, S, D = _dims(q, k, v)
    sc = np.float32(1.0) / np.sqrt(np.float32(D)) if scale is None else np.float32(scale)
    rows = np.ascontiguousarray(rows, dtype=np.int64).reshape(-1, 3)
    out = np.empty((rows.shape[0], D), dtype=np.float32)
    rc = lib().oracle_sdpa_rows_f32(_p(q), _p(k), _p(v), _p(out), B, Hq, Hkv, L, S, D, int(bool(causal)), float(sc),
                                    rows.ctypes.data_as(_c_i64p), rows.shape[0], nthreads or default_threads())
    if rc != 0:
        raise RuntimeError("oracle_sdpa_rows_f32 failed: %d" % rc)
    return out


def sdpa_backward_f32(q, k, v, dout, causal=False, scale=None, mask=None, nthreads=None):
    """Gradients (dq, dk, dv) of sum(sdpa(q, k, v) * dout): the chain rule through the restated forward, accumulated in
    double.  Same shapes and mask conventions as sdpa_f32."""
    q, k, v, dout = _f32(q), _f32(k), _f32(v), _f32(dout)
    B, Hq, Hkv, L, S, D = _dims(q, k, v)
    assert dout.shape == q.shape
    sc = np.float32(1.0) / np.sqrt(np.float32(D)) if scale is None else np.float32(scale)
    if mask is not None and tuple(mask.shape) != (L, S):
        full = np.broadcast_to(mask, (B, Hq, L, S))   # every (batch, head) slice sees its own [L,S] slice
        G = Hq // Hkv
        dq = np.empty(q.shape, dtype=np.float32)
        dk = np.zeros(k.shape, dtype=np.float64)
        dv = np.zeros(v.shape, dtype=np.float64)
        for b in range(B):
            for h in range(Hq):
                hk = h // G
                a, bk, bv = sdpa_backward_f32(q[b:b + 1, h:h + 1], k[b:b + 1, hk:hk + 1], v[b:b + 1, hk:hk + 1],
                                              dout[b:b + 1, h:h + 1], scale=sc, mask=np.ascontiguousarray(full[b, h]),
                                              nthreads=nthreads)
                dq[b, h] = a[0, 0]
                dk[b, hk] += bk[0, 0]
                dv[b, hk] += bv[0, 0]
        return dq, dk.astype(np.float32), dv.astype(np.float32)
    kind, keep, mp = _mask_args(mask, L, S)
    dq = np.empty(q.shape, dtype=np.float32)
    dk = np.zeros(k.shape, dtype=np.float32)
    dv = np.zeros(v.shape, dtype=np.float32)
    rc = lib().oracle_sdpa_backward_f32(_p(q), _p(k), _p(v), _p(dout), _p(dq), _p(dk), _p(dv), B, Hq, Hkv, L, S, D,
                                        int(bool(causal)), float(sc), kind, mp, nthreads or default_threads())
    if rc != 0:
        raise RuntimeError("oracle_sdpa_backward_f32 failed: %d" % rc)
    return dq, dk, dv


def ref_sdpa_f32(q, k, v, causal=False, scale=None, mask=None):
    """tinytorch::function::sdpAttention of the compiled reference (single-threaded, fp32 CPU)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, Hq, Hkv, L, S, D = _dims(q, k, v)
    kind, keep, mp = _mask_args(mask, L, S, any_shape=True)
    mdims = (ctypes.c_int64 * 8)(*(keep.shape if keep is not None else ()))
    out = np.empty(q.shape, dtype=np.float32)
    rc = ref().tt_ref_sdpa_f32(_p(q), _p(k), _p(v), _p(out), B, Hq, Hkv, L, S, D, int(bool(causal)),
                               0 if scale is None else 1, 0.0 if scale is None else float(scale), kind, mp,
                               keep.ndim if keep is not None else 0, mdims)
    if rc != 0:
        raise RuntimeError("tt_ref_sdpa_f32 failed: %d" % rc)
    return out


def ref_sdpa_f32_gqa5d(q, k, v, causal=False):
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, Hq, Hkv, L, S, D = _dims(q, k, v)
    out = np.empty(q.shape, dtype=np.float32)
    rc = ref().tt_ref_sdpa_f32_gqa5d(_p(q), _p(k), _p(v), _p(out), B, Hq, Hkv, L, S, D, int(bool(causal)))
    if rc != 0:
        raise RuntimeError("tt_ref_sdpa_f32_gqa5d failed: %d" % rc)
    return out


def ref_round_trip(x, dtype):
    d = _DTYPES[dtype] if isinstance(dtype, str) else dtype
    x = _f32(x).reshape(-1)
    out = np.empty_like(x)
    ref().tt_ref_round_trip(_p(x), _p(out), x.size, d)
    return out


# ---- row-wise neighbour ops (oracle/fused_oracle.c) ---------------------------------------------------------------

def _dt(dtype):
    return _DTYPES[dtype] if isinstance(dtype, str) else dtype


def _softmax_dims(shape, dim):
    dim = dim % len(shape)
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    inner = int(np.prod(shape[dim + 1:], dtype=np.int64))
    return outer, int(shape[dim]), inner


def rms_norm(x, w=None, eps=1e-8, dtype="f32"):
    """rmsNorm over the last axis; x holds values representable in dtype, the result is rounded to dtype."""
    x = _f32(x)
    w = _f32(w) if w is not None else None
    out = np.empty_like(x)
    dim = x.shape[-1]
    lib().oracle_rms_norm(_p(x), _p(w) if w is not None else None, _p(out), x.size // dim, dim, eps, _dt(dtype))
    return out


def fused_add_rms_norm(inp, residual, w, eps, dtype="f32"):
    """-> (input after, residual after): residual <- input + residual, input <- rmsNorm(residual) * w."""
    a, r, w = _f32(inp).copy(), _f32(residual).copy(), _f32(w)
    dim = a.shape[-1]
    lib().oracle_fused_add_rms_norm(_p(a), _p(r), _p(w), a.size // dim, dim, eps, _dt(dtype))
    return a, r


def silu_mul(x, dtype="f32"):
    x = _f32(x)
    d = x.shape[-1] // 2
    out = np.empty(x.shape[:-1] + (d,), dtype=np.float32)
    lib().oracle_silu_mul(_p(x), _p(out), x.size // (2 * d) if d else 0, d, _dt(dtype))
    return out


def softmax(x, dim=-1, log=False, dtype="f32"):
    x = _f32(x)
    out = np.empty_like(x)
    outer, n, inner = _softmax_dims(x.shape, dim)
    lib().oracle_softmax(_p(x), _p(out), outer, n, inner, int(log), _dt(dtype))
    return out


def softmax_backward(grad, output, dim=-1, log=False, dtype="f32"):
    """Gradient of softmax / logSoftmax along `dim` from the upstream gradient and the forward's output."""
    g, y = _f32(grad), _f32(output)
    assert g.shape == y.shape
    out = np.empty_like(g)
    outer, n, inner = _softmax_dims(g.shape, dim)
    lib().oracle_softmax_backward(_p(g), _p(y), _p(out), outer, n, inner, int(log), _dt(dtype))
    return out


def ref_softmax_backward(grad, output, dim=-1, log=False):
    g, y = _f32(grad), _f32(output)
    out = np.empty_like(g)
    outer, n, inner = _softmax_dims(g.shape, dim)
    rc = ref().tt_ref_softmax_backward(_p(g), _p(y), _p(out), outer, n, inner, int(log))
    assert rc == 0
    return out


def ref_rms_norm(x, w=None, eps=1e-8):
    x = _f32(x)
    w = _f32(w) if w is not None else None
    out = np.empty_like(x)
    dim = x.shape[-1]
    rc = ref().tt_ref_rms_norm(_p(x), _p(w) if w is not None else None, _p(out), x.size // dim, dim, eps)
    assert rc == 0
    return out


def ref_fused_add_rms_norm(inp, residual, w, eps):
    a, r, w = _f32(inp).copy(), _f32(residual).copy(), _f32(w)
    dim = a.shape[-1]
    rc = ref().tt_ref_fused_add_rms_norm(_p(a), _p(r), _p(w), a.size // dim, dim, eps)
    assert rc == 0
    return a, r


def ref_silu_mul(x):
    x = _f32(x)
    d = x.shape[-1] // 2
    out = np.empty(x.shape[:-1] + (d,), dtype=np.float32)
    rc = ref().tt_ref_silu_mul(_p(x), _p(out), x.size // (2 * d), d)
    assert rc == 0
    return out


def ref_softmax(x, dim=-1, log=False):
    x = _f32(x)
    out = np.empty_like(x)
    outer, n, inner = _softmax_dims(x.shape, dim)
    rc = ref().tt_ref_softmax(_p(x), _p(out), outer, n, inner, int(log))
    assert rc == 0
    return out


def linear(x, w, bias=None, dtype="f32"):
    """x [M,K] . w [N,K]^T + bias [N] in the reference's loop order; the result rounded to dtype."""
    x, w = _f32(x), _f32(w)
    b = _f32(bias) if bias is not None else None
    M, K = x.shape
    N = w.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    lib().oracle_linear(_p(x), _p(w), _p(b) if b is not None else None, _p(out), M, N, K, _dt(dtype))
    return out


def _matmul_dims(a, b, transA, transB):
    K, M = a.shape if transA else a.shape[::-1]
    Kb, N = b.shape[::-1] if transB else b.shape
    assert K == Kb
    return M, N, K


def matmul(a, b, transA=False, transB=False, bias=None, dtype="f32"):
    """op(a) . op(b) + bias in the reference's loop order: a [M,K] ([K,M] with transA), b [K,N] ([N,K] with transB)."""
    a, b = _f32(a), _f32(b)
    bs = _f32(bias) if bias is not None else None
    M, N, K = _matmul_dims(a, b, transA, transB)
    out = np.empty((M, N), dtype=np.float32)
    lib().oracle_matmul(_p(a), _p(b), _p(bs) if bs is not None else None, _p(out), M, N, K, int(transA), int(transB), _dt(dtype))
    return out


def matmul_nd(a, b, transA=False, transB=False, bias=None, dtype="f32"):
    """op::matmul with the reference's batch and 1-D rules (src/Operation/OpLinalg.cpp:52-241): a 1-D a is a row vector,
    a 1-D b a column vector (their flags ignored, :63-72); leading dimensions broadcast (:84-89); every batch entry is
    the 2-D product of the operands' slices at that index (the CPU path's loop, :205-223: an operand whose dimension is 1
    stays at its only slice); the added dimensions are dropped from a 2-D result (:221-239)."""
    a, b = _f32(a), _f32(b)
    assert a.ndim >= 1 and b.ndim >= 1
    prepend_a, append_b = a.ndim == 1, b.ndim == 1
    if prepend_a:
        a, transA = a[None, :], False
    if append_b:
        b, transB = b[:, None], False
    batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    M = a.shape[-1] if transA else a.shape[-2]
    N = b.shape[-2] if transB else b.shape[-1]
    ea = np.broadcast_to(a, batch + a.shape[-2:])
    eb = np.broadcast_to(b, batch + b.shape[-2:])
    out = np.empty(batch + (M, N), dtype=np.float32)
    for idx in np.ndindex(*batch):
        out[idx] = matmul(np.ascontiguousarray(ea[idx]), np.ascontiguousarray(eb[idx]), transA, transB, bias, dtype)
    if append_b:
        out = out.reshape(() if prepend_a else (M,))
    elif prepend_a and not batch:
        out = out.reshape(N)
    return out


def ref_matmul(a, b, transA=False, transB=False, bias=None):
    """op::matmul of the compiled reference (fp32, CPU)."""
    a, b = _f32(a), _f32(b)
    bs = _f32(bias) if bias is not None else None
    M, N, K = _matmul_dims(a, b, transA, transB)
    out = np.empty((M, N), dtype=np.float32)
    rc = ref().tt_ref_matmul(_p(a), _p(b), _p(bs) if bs is not None else None, _p(out), M, N, K, int(transA), int(transB))
    assert rc == 0
    return out


def ref_linear(x, w, bias=None):
    x, w = _f32(x), _f32(w)
    b = _f32(bias) if bias is not None else None
    M, K = x.shape
    N = w.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    rc = ref().tt_ref_linear(_p(x), _p(w), _p(b) if b is not None else None, _p(out), M, N, K)
    assert rc == 0
    return out
