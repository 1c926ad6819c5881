"""A generation step (KV-cache append, per-batch key counts, attention) recorded into a HIP graph and replayed.

The C ABI only enqueues kernels on the caller's stream and reads positions / key counts from device memory, so a
serving loop can record one step and replay it per token.  Every replay is checked against the eager result, with the
program's own eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, max_abs_err, to_device
from tinytorch_amd import kvCacheAppend, sdpAttention

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,Hq,Hkv,Smax", [(4, 8, 2, 640), (1, 32, 8, 4096)])  # unsplit; split cache + merge kernel
def test_decode_step_in_a_graph(B, Hq, Hkv, Smax):
    D, dtype, steps = 128, "bf16", 4
    kh, kb = oracle.round_to(oracle.randn(501, 1, (B, Hkv, Smax, D)), dtype)
    vh, vb = oracle.round_to(oracle.randn(501, 2, (B, Hkv, Smax, D)), dtype)
    kd, vd = to_device(kh, kb, dtype), to_device(vh, vb, dtype)
    start = np.array([(97 * (b + 1)) % (Smax // 2) + 3 for b in range(B)], np.int32)
    pmax = int(start.max())
    kc, vc = torch.zeros_like(kd), torch.zeros_like(vd)
    kvCacheAppend(kc, vc, kd[:, :, :pmax], vd[:, :, :pmax], 0)

    # static buffers of the recorded step
    lens = torch.from_numpy(start.copy()).cuda()          # rows filled so far, advanced on the device
    q_buf = torch.zeros(B, Hq, 1, D, dtype=torch.bfloat16, device="cuda")
    kn_buf = torch.zeros(B, Hkv, 1, D, dtype=torch.bfloat16, device="cuda")
    vn_buf = torch.zeros_like(kn_buf)
    out_buf = torch.zeros_like(q_buf)

    def step():
        kvCacheAppend(kc, vc, kn_buf, vn_buf, lens)
        lens.add_(1)
        out_buf.copy_(sdpAttention(q_buf, kc, vc, kvLens=lens))

    def feed(t, cur):
        qh, qb = oracle.round_to(oracle.randn(600 + t, 0, (B, Hq, 1, D)), dtype)
        q_buf.copy_(to_device(qh, qb, dtype))
        kn_buf.copy_(torch.stack([kd[b, :, cur[b]:cur[b] + 1] for b in range(B)]))
        vn_buf.copy_(torch.stack([vd[b, :, cur[b]:cur[b] + 1] for b in range(B)]))
        return qh

    # one eager step first: it also performs the library's one-time set-up outside the capture
    cur = start.copy()
    qh = feed(0, cur)
    step()
    cur += 1
    torch.cuda.synchronize()
    for b in range(B):
        exp = oracle.sdpa_f32(qh[b:b + 1], kh[b:b + 1, :, :cur[b]], vh[b:b + 1, :, :cur[b]])
        assert max_abs_err(out_buf[b:b + 1], exp) <= TOL[dtype]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    qh = feed(1, cur)          # the capture itself does not execute: feed, capture, then replay this same step
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step()
    for t in range(1, 1 + steps):
        if t > 1:
            qh = feed(t, cur)
        graph.replay()
        cur += 1
        torch.cuda.synchronize()
        assert np.array_equal(lens.cpu().numpy(), cur)
        for b in range(B):
            exp = oracle.sdpa_f32(qh[b:b + 1], kh[b:b + 1, :, :cur[b]], vh[b:b + 1, :, :cur[b]])
            assert max_abs_err(out_buf[b:b + 1], exp) <= TOL[dtype], (t, b)
        # eager work between the replays: the same attention without the graph gives the same bits
        eager = sdpAttention(q_buf, kc, vc, kvLens=lens)
        torch.cuda.synchronize()
        assert torch.equal(eager, out_buf)
    for b in range(B):
        assert torch.equal(kc[b, :, :cur[b]], kd[b, :, :cur[b]])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_forward_and_backward_in_a_graph(dtype):
    """A training-style step (attention forward, then its backward) recorded once and replayed on new inputs: both
    calls only enqueue kernels and use caller-provided scratch, so every replay reproduces the eager bits.  At this
    shape the dk/dv kernels split their query streams: the partial sums in scratch and the kernel that adds them are
    part of the recorded step."""
    import ctypes
    from tinytorch_amd import _capi, build_backward_params, build_params
    B, Hq, Hkv, N, D = 2, 8, 2, 384, 128
    gen = torch.Generator(device="cuda").manual_seed(77)
    mk = lambda *shape: torch.randn(*shape, device="cuda", generator=gen).to(dtype)
    q, k, v, go = mk(B, Hq, N, D), mk(B, Hkv, N, D), mk(B, Hkv, N, D), mk(B, Hq, N, D)
    out, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    L = _capi.lib()
    fp = build_params(q, k, v, out, True)
    bp = build_backward_params(q, k, v, out, go, dq, dk, dv, True)
    nbytes = L.ttsdpa_backward_workspace_bytes(ctypes.byref(bp))
    assert nbytes > B * Hq * N * 8   # more than the statistics: partial dk / dv
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")

    def step():
        st = torch.cuda.current_stream().cuda_stream
        assert L.ttsdpa_forward(ctypes.byref(fp), None, 0, st) == 0
        assert L.ttsdpa_backward(ctypes.byref(bp), ws.data_ptr(), nbytes, st) == 0

    step()   # eager once: one-time set-up of the kernels happens outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step()
    for t in range(3):
        for buf in (q, k, v, go):
            buf.copy_(mk(*buf.shape))
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in (out, dq, dk, dv)]
        for x in (out, dq, dk, dv):
            x.zero_()
        step()   # the same step eagerly
        torch.cuda.synchronize()
        for a, b in zip(got, (out, dq, dk, dv)):
            assert torch.equal(a, b), t
