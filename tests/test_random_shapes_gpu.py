"""Seeded random call shapes through ttsdpa_forward against the oracle: every route, ragged sizes, grouped heads,
causal / masks / per-batch key counts.  The shapes are drawn once from a fixed seed, so a failure names its case."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, make_inputs, max_abs_err, route_of, to_device
from tinytorch_amd import sdpAttention

pytestmark = pytest.mark.gpu


def _head_dim(rng, dtype, other, limit):
    """A head size: one of the kernels' own, or (other) any size their zero-column variants take, up to `limit`."""
    if not other:
        return None
    step = 4 if dtype == "f32" else 8
    top = min(limit, 128) if dtype == "f32" else limit
    return int(rng.randint(1, top // step + 1)) * step


def _cases(other=False):
    rng = np.random.RandomState(20250115 if other else 20240607)
    out = []
    for i in range(40 if other else 48):
        dtype = ["bf16", "f16", "f32"][rng.randint(3)]
        D = [128, 128, 128, 64, 32, 80][rng.randint(6)]
        D = _head_dim(rng, dtype, other, 256) or D
        Hkv = int(rng.randint(1, 4))
        G = [1, 1, 2, 4, 7][rng.randint(5)]
        B = int(rng.randint(1, 4))
        kind = ["prefill", "prefill", "decode", "short"][rng.randint(4)]
        if kind == "prefill":
            L = int(rng.randint(129, 700))
            S = L if rng.rand() < 0.5 else int(rng.randint(1, 900))
        elif kind == "decode":
            L = int(rng.randint(1, 4))
            S = int(rng.randint(1, 3000))
            G = min(G, 16 // L)
        else:
            L = int(rng.randint(1, 129))
            S = int(rng.randint(1, 400))
        extra = ["none", "none", "causal", "causal", "boolmask", "addmask", "kvlen"][rng.randint(7)]
        out.append((i + (100 if other else 0), dtype, B, Hkv * G, Hkv, L, S, D, extra))
    return out


@pytest.mark.parametrize("case", _cases() + _cases(other=True), ids=lambda c: "%d-%s-B%d-H%d/%d-L%d-S%d-D%d-%s" % c)
def test_random_shape(case):
    i, dtype, B, Hq, Hkv, L, S, D, extra = case
    host, dev = make_inputs(3000 + i, B, Hq, Hkv, L, S, D, dtype)
    kw_dev, kw_host = {}, {}
    if extra == "causal":
        kw_dev["isCausal"] = True
        kw_host["causal"] = True
    elif extra == "boolmask":
        m = (np.random.RandomState(i).rand(B, 1, L, S) > 0.4).astype(np.uint8)
        m[..., 0] = 1  # no row without a visible key
        kw_dev["attnMask"] = torch.from_numpy(m).cuda().bool()
        kw_host["mask"] = m
    elif extra == "addmask":
        m, bits = oracle.round_to(oracle.randn(4000 + i, 5, (Hq, 1, S)), dtype)
        kw_dev["attnMask"] = to_device(m, bits, dtype)
        kw_host["mask"] = m
    if extra == "kvlen":
        lens = np.random.RandomState(i).randint(1, S + 1, size=B).astype(np.int32)
        out = sdpAttention(*dev, kvLens=torch.from_numpy(lens).cuda())
        torch.cuda.synchronize()
        for b in range(B):
            exp = oracle.sdpa_f32(host[0][b:b + 1], host[1][b:b + 1, :, :lens[b]], host[2][b:b + 1, :, :lens[b]])
            assert max_abs_err(out[b:b + 1], exp) <= TOL[dtype], (route_of(*dev), b)
        return
    out = sdpAttention(*dev, **kw_dev)
    torch.cuda.synchronize()
    exp = oracle.sdpa_f32(*host, **kw_host)
    assert max_abs_err(out, exp) <= TOL[dtype], route_of(*dev, causal=extra == "causal")


def _backward_cases(other=False):
    rng = np.random.RandomState(20250116 if other else 20240911)
    out = []
    for i in range(32 if other else 40):
        dtype = ["bf16", "f16", "f32"][rng.randint(3)]
        D = [128, 128, 64, 64, 32, 80][rng.randint(6)]
        D = _head_dim(rng, dtype, other, 128) or D
        Hkv = int(rng.randint(1, 3))
        G = [1, 1, 2, 4, 3][rng.randint(5)]
        B = int(rng.randint(1, 3))
        L = int(rng.randint(1, 330))
        S = L if rng.rand() < 0.4 else int(rng.randint(1, 400))
        extra = ["none", "causal", "causal-br", "boolmask", "addmask", "kvlen", "boolmask4"][rng.randint(7)]
        if extra == "boolmask4":
            S = (S + 3) // 4 * 4   # keys readable four at a time: the MFMA pair's masks
        out.append((i + (100 if other else 0), dtype, B, Hkv * G, Hkv, L, S, D, extra))
    return out


@pytest.mark.parametrize("case", _backward_cases() + _backward_cases(other=True), ids=lambda c: "%d-%s-B%d-H%d/%d-L%d-S%d-D%d-%s" % c)
def test_random_backward_shape(case):
    """The same idea for ttsdpa_backward: both kernel families, ragged tiles on both sides, grouped heads, both causal
    alignments, masks, per-batch key counts — against the oracle's gradients."""
    from gpu_util import backward_route_of, grad_err
    from tinytorch_amd import sdpAttentionBackward
    i, dtype, B, Hq, Hkv, L, S, D, extra = case
    host, dev = make_inputs(5000 + i, B, Hq, Hkv, L, S, D, dtype)
    go_h, go_b = oracle.round_to(oracle.randn(5000 + i, 9, host[0].shape), dtype)
    go = to_device(go_h, go_b, dtype)
    kw, mask_h, lens = {}, None, None
    if extra == "causal":
        kw["isCausal"] = True
        mask_h = np.arange(S)[None, :] <= np.arange(L)[:, None]
        if S < L:
            mask_h = mask_h.copy()   # rows past S see every key: nothing to fix, the tril covers it
    elif extra == "causal-br":
        kw.update(isCausal=True, causalAlign="bottom-right")
        mask_h = np.arange(S)[None, :] <= np.arange(L)[:, None] + max(0, S - L)
    elif extra in ("boolmask", "boolmask4"):
        mask_h = np.random.RandomState(i).rand(B, 1, L, S) > 0.4
        mask_h[..., 0] = True
        kw["attnMask"] = torch.from_numpy(mask_h).cuda()
    elif extra == "addmask":
        mask_h, bits = oracle.round_to(oracle.randn(6000 + i, 5, (Hq, 1, S)), dtype)
        kw["attnMask"] = to_device(mask_h, bits, dtype)
    elif extra == "kvlen":
        lens = np.random.RandomState(i).randint(1, S + 1, size=B).astype(np.int32)
        kw["kvLens"] = torch.from_numpy(lens).cuda()
    out = sdpAttention(*dev, **kw)
    dq, dk, dv = sdpAttentionBackward(go, *dev, out, **kw)
    torch.cuda.synchronize()
    if lens is not None:
        for b in range(B):
            n = int(lens[b])
            eq, ek, ev = oracle.sdpa_backward_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n], go_h[b:b + 1])
            assert grad_err(dq[b:b + 1], eq) <= TOL[dtype] and grad_err(dk[b:b + 1, :, :n], ek) <= TOL[dtype]
            assert grad_err(dv[b:b + 1, :, :n], ev) <= TOL[dtype]
            assert torch.all(dk[b, :, n:] == 0) and torch.all(dv[b, :, n:] == 0)
        return
    eq, ek, ev = oracle.sdpa_backward_f32(*host, go_h, mask=mask_h)
    for name, got, exp in (("dq", dq, eq), ("dk", dk, ek), ("dv", dv, ev)):
        assert grad_err(got, exp) <= TOL[dtype], name
