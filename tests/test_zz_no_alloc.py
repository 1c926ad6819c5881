"""ttsdpa_decode_static: the decode entry point that allocates nothing (its split-KV partial records live in a buffer that
is part of the library's device image) against ttsdpa_decode with caller scratch, through the C ABI.  Two calls in a
row, the second on a smaller input, so that what the first call left in the shared buffer is there for the second."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, make_inputs, to_host_f32
from tinytorch_amd import _capi, build_params

pytestmark = pytest.mark.gpu


def _both(B, Hq, Hkv, L, S, D, dtype, seed):
    host, dev = make_inputs(seed, B, Hq, Hkv, L, S, D, dtype)
    lib = _capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    out_ws = torch.empty_like(dev[0])
    p = build_params(*dev, out_ws, False)
    nbytes = lib.ttsdpa_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    assert lib.ttsdpa_decode(ctypes.byref(p), ws.data_ptr(), nbytes, stream) == 0
    out_static = torch.full_like(dev[0], float("nan"))
    p2 = build_params(*dev, out_static, False)
    rc = lib.ttsdpa_decode_static(ctypes.byref(p2), stream)
    assert rc == 0, _capi.status_string(rc)
    torch.cuda.synchronize()
    return host, out_ws, out_static, nbytes


def test_static_scratch_decode_matches_decode_twice_in_a_row():
    # first call: one batch entry, long cache -> many splits, about 1 MB of partial records
    host, a, b, n1 = _both(1, 8, 2, 1, 16384, 128, "bf16", 31)
    print("first call: scratch %d bytes" % n1, flush=True)
    assert n1 > 0 and torch.equal(a.view(torch.int16), b.view(torch.int16))
    err = float(np.abs(to_host_f32(b) - oracle.sdpa_f32(*host)).max())
    assert err <= TOL["bf16"]
    # second call, smaller: fewer splits, fewer rows; the buffer still holds the first call's records
    host, a, b, n2 = _both(2, 4, 2, 1, 2048, 128, "bf16", 32)
    print("second call: scratch %d bytes" % n2, flush=True)
    assert 0 < n2 < n1 and torch.equal(a.view(torch.int16), b.view(torch.int16))
    err = float(np.abs(to_host_f32(b) - oracle.sdpa_f32(*host)).max())
    assert err <= TOL["bf16"]
    # and a call that needs no scratch at all (enough (batch, head) pairs to run unsplit), fp16, head_dim 64
    host, a, b, n3 = _both(64, 8, 8, 1, 512, 64, "f16", 33)
    assert n3 == 0 and torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_static_scratch_decode_allocates_nothing_and_replays_in_a_graph():
    """The property the entry point exists for.  After a warm call (the library looks up its buffer's address once per
    device) further calls leave the device's free memory unchanged, and a call recorded into a HIP graph — where an
    allocation would fail the capture — replays to what ttsdpa_decode gives with caller scratch, replay after replay,
    with eager work and synchronisations between the replays."""
    B, Hq, Hkv, S, D = 1, 8, 2, 16384, 128   # many splits: the partial records are in use
    host, dev = make_inputs(41, B, Hq, Hkv, 1, S, D, "bf16")
    lib = _capi.lib()
    out_ws, out_static = torch.empty_like(dev[0]), torch.empty_like(dev[0])
    p_ws, p_static = build_params(*dev, out_ws, False), build_params(*dev, out_static, False)
    nbytes = lib.ttsdpa_workspace_bytes(ctypes.byref(p_ws))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert nbytes > 0 and lib.ttsdpa_decode(ctypes.byref(p_ws), ws.data_ptr(), nbytes, stream) == 0
    assert lib.ttsdpa_decode_static(ctypes.byref(p_static), stream) == 0   # warm call
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(8):
        assert lib.ttsdpa_decode_static(ctypes.byref(p_static), stream) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, "device memory changed across ttsdpa_decode_static calls: %d -> %d" % (free0, free1)
    assert torch.equal(out_ws.view(torch.int16), out_static.view(torch.int16))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.ttsdpa_decode_static(ctypes.byref(p_static), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _capi.status_string(rc)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        qh, qb = oracle.round_to(oracle.randn(50 + rep, 0, (B, Hq, 1, D)), "bf16")
        dev[0].copy_(torch.from_numpy(qb.view(np.int16)).cuda().view(torch.bfloat16))   # new queries in the recorded buffer
        out_static.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        assert lib.ttsdpa_decode(ctypes.byref(p_ws), ws.data_ptr(), nbytes, stream) == 0   # eager, caller scratch
        torch.cuda.synchronize()
        assert torch.equal(out_ws.view(torch.int16), out_static.view(torch.int16)), "replay %d" % rep
        err = float(np.abs(to_host_f32(out_static) - oracle.sdpa_f32(qh, host[1], host[2])).max())
        assert err <= TOL["bf16"]
