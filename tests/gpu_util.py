"""Helpers for the GPU parity tests: seeded inputs shared bit-for-bit by the HIP path and the CPU oracle, and thin
callers of the C ABI entry points (include/ttsdpa.h) on torch-owned device memory."""
import ctypes

import numpy as np
import torch

import oracle
from tinytorch_amd import _capi
from tinytorch_amd.function import build_params

TORCH_DTYPE = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
TOL = {"f32": 1e-4, "f16": 2e-2, "bf16": 2e-2}  # max-abs-error bars of the north-star statement


def to_device(vals_f32, bits, dtype):
    """Device tensor of `dtype` holding exactly the rounded values the oracle sees."""
    if dtype == "f32":
        return torch.from_numpy(np.ascontiguousarray(vals_f32)).cuda()
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda()
    return t.view(TORCH_DTYPE[dtype])


def make_inputs(seed, B, Hq, Hkv, L, S, D, dtype, mul=1.0):
    """-> (host fp32 values after rounding to dtype) x3, (device tensors) x3"""
    host, dev = [], []
    for stream, shape in enumerate(((B, Hq, L, D), (B, Hkv, S, D), (B, Hkv, S, D))):
        x = oracle.randn(seed, stream, shape, mul)
        vals, bits = oracle.round_to(x, dtype)
        host.append(vals)
        dev.append(to_device(vals, bits, dtype))
    return host, dev


def to_host_f32(t):
    return t.detach().float().cpu().numpy()


def call(entry, q, k, v, causal=False, mask=None, scale=None, out=None, kv_lens=None, align="top-left", block_table=None):
    """Run one C ABI entry point ("forward" | "prefill" | "decode" | "general") -> (status, out tensor)."""
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    p = build_params(q, k, v, out, causal, mask, scale, kv_lens, align, block_table)
    L = _capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    ws, nbytes = None, 0
    if entry in ("forward", "decode"):
        nbytes = L.ttsdpa_workspace_bytes(ctypes.byref(p))
        if nbytes:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    wsp = ws.data_ptr() if ws is not None else None
    if entry == "forward":
        rc = L.ttsdpa_forward(ctypes.byref(p), wsp, nbytes, stream)
    elif entry == "decode":
        rc = L.ttsdpa_decode(ctypes.byref(p), wsp, nbytes, stream)
    elif entry == "prefill":
        rc = L.ttsdpa_prefill(ctypes.byref(p), stream)
    else:
        rc = L.ttsdpa_general(ctypes.byref(p), stream)
    torch.cuda.synchronize()
    return rc, out


def route_of(q, k, v, causal=False, mask=None, scale=None, out=None, kv_lens=None, align="top-left", block_table=None):
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    rc, r = _capi.plan(build_params(q, k, v, out, causal, mask, scale, kv_lens, align, block_table))
    assert rc == 0
    return _capi.ROUTE_NAMES[r]


def max_abs_err(out_dev, expect):
    y = to_host_f32(out_dev)
    assert y.shape == expect.shape
    assert np.isfinite(y).all(), "non-finite values in the GPU result"
    return float(np.abs(y.astype(np.float64) - expect.astype(np.float64)).max())


def backward_call(q, k, v, out, dout, causal=False, mask=None, scale=None, kv_lens=None, align="top-left", grads=None,
                  ws_bytes=None):
    """ttsdpa_backward through the C ABI -> (status, (dq, dk, dv))."""
    from tinytorch_amd.function import build_backward_params
    if grads is None:
        grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    bp = build_backward_params(q, k, v, out, dout, grads[0], grads[1], grads[2], causal, mask, scale, kv_lens, align)
    L = _capi.lib()
    nbytes = L.ttsdpa_backward_workspace_bytes(ctypes.byref(bp)) if ws_bytes is None else ws_bytes
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
    rc = L.ttsdpa_backward(ctypes.byref(bp), ws.data_ptr() if nbytes else None, nbytes, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc, grads


def backward_route_of(q, k, v, out, dout, causal=False, mask=None, scale=None, kv_lens=None, align="top-left"):
    from tinytorch_amd.function import build_backward_params
    g = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    bp = build_backward_params(q, k, v, out, dout, g[0], g[1], g[2], causal, mask, scale, kv_lens, align)
    r = ctypes.c_int(-1)
    assert _capi.lib().ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(r)) == 0
    return _capi.ROUTE_NAMES[r.value]


def grad_err(got_dev, expect):
    """Max abs error of a gradient, in units of max(1, largest expected magnitude): the forward's bar applied to a
    tensor whose entries are sums over many rows and exceed 1."""
    y = to_host_f32(got_dev)
    assert y.shape == expect.shape
    assert np.isfinite(y).all(), "non-finite values in the GPU gradient"
    return float(np.abs(y.astype(np.float64) - expect.astype(np.float64)).max() / max(1.0, float(np.abs(expect).max())))
