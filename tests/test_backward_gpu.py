"""Attention backward through the C ABI (ttsdpa_backward) against the oracle's gradients on the same seeded inputs.

The reference has no attention backward (reference src/Function/FuncNNLayer.h:267 is NOT_IMPLEMENTED), so the oracle's
gradients are pinned by differences, closed forms and invariants (tests/test_oracle_backward.py) rather than against
reference vectors.  Bars: the forward's (fp32 1e-4, fp16/bf16 2e-2), in units of max(1, largest expected magnitude) —
gradient entries are sums over many rows.  `out` handed to the backward is what the GPU forward produced."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import (TOL, TORCH_DTYPE, backward_call, backward_route_of, call, grad_err, make_inputs, to_device,
                      to_host_f32)
from tinytorch_amd import _capi, build_backward_params, sdpAttention, sdpAttentionBackward

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def upstream(seed, shape, dtype):
    vals, bits = oracle.round_to(oracle.randn(seed, 7, shape), dtype)
    return vals, to_device(vals, bits, dtype)


def check(case_name, host, dev, dtype, causal=False, mask_h=None, mask_d=None, scale=None, kv_lens=None, align="top-left",
          oracle_mask=None, route=None):
    say("backward", case_name)
    q, k, v = dev
    go_h, go = upstream(hash(case_name) % 1000, q.shape, dtype)
    rc, out = call("forward", q, k, v, causal=causal, mask=mask_d, scale=scale, kv_lens=kv_lens, align=align)
    assert rc == 0
    if route is not None:
        assert backward_route_of(q, k, v, out, go, causal, mask_d, scale, kv_lens, align) == route
    rc, (dq, dk, dv) = backward_call(q, k, v, out, go, causal, mask_d, scale, kv_lens, align)
    assert rc == 0
    om = oracle_mask if oracle_mask is not None else mask_h
    ocausal = causal and oracle_mask is None
    eq, ek, ev = oracle.sdpa_backward_f32(host[0], host[1], host[2], go_h, causal=ocausal, scale=scale, mask=om)
    for name, got, exp in (("dq", dq, eq), ("dk", dk, ek), ("dv", dv, ev)):
        err = grad_err(got, exp)
        assert err <= TOL[dtype], (name, err)


GENERAL_CASES = [
    # B, Hq, Hkv, L, S, D, dtype, causal
    (1, 1, 1, 3, 5, 8, "f32", False),
    (2, 4, 4, 33, 33, 64, "f32", True),
    (2, 8, 2, 70, 130, 40, "f32", False),      # grouped heads, head_dim not a multiple of 64
    (1, 4, 2, 65, 20, 96, "f32", True),        # L > S, top-left causal: rows past S see every key
    (1, 2, 1, 17, 200, 256, "f32", False),     # the largest head_dim
    (2, 4, 2, 70, 45, 160, "f32", True),       # head_dim in (128, 256]: eight lanes per row, 16-row tiles
    (1, 6, 2, 40, 90, 136, "bf16", True),
    (1, 2, 2, 33, 64, 256, "f16", False),
    (2, 4, 2, 50, 77, 64, "bf16", True),
    (2, 4, 2, 50, 77, 128, "f16", False),
    (1, 6, 3, 129, 64, 32, "bf16", False),
]


@pytest.mark.parametrize("case", GENERAL_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-c%d" % c)
def test_backward_against_oracle(case):
    B, Hq, Hkv, L, S, D, dtype, causal = case
    host, dev = make_inputs(4000 + L + S + D, B, Hq, Hkv, L, S, D, dtype)
    check("plain-%s" % (case,), host, dev, dtype, causal=causal)


MFMA_CASES = [
    # B, Hq, Hkv, L, S, D, dtype, causal ("br" = bottom-right aligned)
    (2, 8, 2, 256, 256, 128, "bf16", True),
    (1, 4, 4, 200, 333, 64, "f16", False),        # ragged last tiles on both sides
    (2, 6, 2, 130, 70, 128, "f16", True),         # L > S, top-left: rows past S see every key
    (1, 8, 8, 64, 500, 128, "bf16", "br"),        # a chunk of 64 queries at the end of 500 keys
    (2, 4, 1, 96, 96, 64, "bf16", True),          # four heads per KV head, head_dim 64
    (1, 2, 2, 1, 129, 128, "bf16", False),        # one query row
    (1, 2, 1, 300, 17, 64, "f16", "br"),          # more queries than keys, bottom-right: offset 0
    (3, 4, 2, 33, 257, 128, "f16", False),
    # fp32 tensors: the fp32 matrix-core pair
    (2, 8, 2, 256, 256, 128, "f32", True),
    (1, 4, 4, 200, 333, 64, "f32", False),
    (2, 6, 2, 130, 70, 128, "f32", True),
    (1, 8, 8, 64, 500, 128, "f32", "br"),
    (2, 4, 1, 96, 96, 64, "f32", True),
    (1, 2, 2, 1, 129, 128, "f32", False),
    (1, 2, 1, 300, 17, 64, "f32", "br"),
    (3, 4, 2, 33, 257, 128, "f32", False),
]


@pytest.mark.parametrize("case", MFMA_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-%s" % c)
def test_backward_mfma_against_oracle(case):
    B, Hq, Hkv, L, S, D, dtype, causal = case
    host, dev = make_inputs(4300 + L + S + D, B, Hq, Hkv, L, S, D, dtype)
    if causal == "br":
        m = np.arange(S)[None, :] <= np.arange(L)[:, None] + max(0, S - L)
        check("mfma-%s" % (case,), host, dev, dtype, causal=True, align="bottom-right", oracle_mask=m, route="prefill")
    else:
        check("mfma-%s" % (case,), host, dev, dtype, causal=causal, route="prefill")


PADDED_CASES = [
    # head sizes between the matrix-core kernels' (64, 128): the register-staged pair of the next one up, zero columns
    (2, 4, 2, 150, 150, 80, "bf16", True),
    (1, 4, 4, 200, 333, 40, "f16", False),
    (2, 6, 2, 130, 70, 96, "bf16", True),
    (1, 8, 2, 64, 500, 112, "f16", "br"),
    (2, 2, 1, 96, 96, 8, "bf16", True),
    (1, 2, 2, 1, 129, 120, "bf16", False),
    (1, 4, 1, 300, 17, 24, "f16", "br"),
    (2, 4, 2, 260, 260, 72, "bf16", "mask"),
    (2, 4, 2, 160, 300, 104, "f16", "kvlen"),
    # fp32: multiples of 4 up to 128 on the fp32 matrix-core pair
    (2, 4, 2, 150, 150, 40, "f32", True),
    (1, 4, 4, 100, 233, 100, "f32", False),
    (1, 2, 1, 70, 300, 20, "f32", "br"),
    (2, 4, 2, 130, 260, 96, "f32", "mask"),
    (2, 2, 2, 90, 200, 4, "f32", "kvlen"),
]


@pytest.mark.parametrize("case", PADDED_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-%s" % c)
def test_backward_mfma_head_sizes_between_the_kernels(case):
    B, Hq, Hkv, L, S, D, dtype, mode = case
    print("backward, padded head_dim", case, flush=True)
    host, dev = make_inputs(4700 + L + S + D, B, Hq, Hkv, L, S, D, dtype)
    name = "padded-%s" % (case,)
    if mode == "br":
        m = np.arange(S)[None, :] <= np.arange(L)[:, None] + max(0, S - L)
        check(name, host, dev, dtype, causal=True, align="bottom-right", oracle_mask=m, route="prefill")
    elif mode == "mask":
        m = np.random.default_rng(D).random((Hq, L, S)) < 0.7
        m[..., 0] = True
        check(name, host, dev, dtype, mask_h=m, mask_d=torch.from_numpy(m).cuda(), route="prefill")
    elif mode == "kvlen":
        lens = np.array([S, 77], np.int32)
        kv = torch.from_numpy(lens).cuda()
        m = (np.arange(S)[None, None, :] < lens[:, None, None]) & (np.arange(S)[None, None, :] <= np.arange(L)[None, :, None] + np.maximum(0, lens - L)[:, None, None])
        check(name, host, dev, dtype, causal=True, kv_lens=kv, align="bottom-right", oracle_mask=m[:, None], route="prefill")
    else:
        check(name, host, dev, dtype, causal=mode, route="prefill")


def test_backward_mfma_padded_head_size_touches_its_columns_only():
    # q, k, v, out, dout are views of wider rows whose other columns hold NaN; the gradients are views whose other columns
    # keep a sentinel
    B, Hq, Hkv, L, S, D, W = 1, 4, 2, 140, 200, 80, 128
    host, dev = make_inputs(4801, B, Hq, Hkv, L, S, D, "bf16")
    go_h, go_b = oracle.round_to(oracle.randn(4801, 7, host[0].shape), "bf16")
    go = to_device(go_h, go_b, "bf16")
    out = sdpAttention(*dev, isCausal=True)

    def widen(t, fill):
        w = torch.full(t.shape[:-1] + (W,), fill, dtype=t.dtype, device="cuda")
        w[..., :D] = t
        return w

    wide = [widen(t, float("nan"))[..., :D] for t in (*dev, out, go)]
    gw = [torch.full(t.shape[:-1] + (W,), 7.0, dtype=t.dtype, device="cuda") for t in dev]
    rc, grads = backward_call(wide[0], wide[1], wide[2], wide[3], wide[4], causal=True, grads=tuple(g[..., :D] for g in gw))
    assert rc == 0
    exp = oracle.sdpa_backward_f32(*host, go_h, causal=True)
    for g, w, e in zip(grads, gw, exp):
        assert grad_err(g, e) <= TOL["bf16"] and bool((w[..., D:] == 7.0).all())


def test_backward_mfma_properties_at_size():
    """Config 3's shape (B2 32q/8kv 4096 x 4096 x 128 bf16, causal), where the oracle would take minutes: the gradients are
    linear in dout (doubling it doubles them exactly: every product has one factor from dout), the columns of dk sum to ~0
    (softmax ignores a shift common to all keys), and a sample of dq / dk / dv rows agrees with the vector-ALU kernels run
    on fp32 copies of the same tensors."""
    B, Hq, Hkv, N, D = 2, 32, 8, 4096, 128
    gen = torch.Generator(device="cuda").manual_seed(21)
    q = torch.randn(B, Hq, N, D, device="cuda", generator=gen).bfloat16()
    k = torch.randn(B, Hkv, N, D, device="cuda", generator=gen).bfloat16()
    v = torch.randn(B, Hkv, N, D, device="cuda", generator=gen).bfloat16()
    go = torch.randn(B, Hq, N, D, device="cuda", generator=gen).bfloat16()
    out = sdpAttention(q, k, v, isCausal=True)
    assert backward_route_of(q, k, v, out, go, True) == "prefill"
    dq, dk, dv = sdpAttentionBackward(go, q, k, v, out, isCausal=True)
    dq2, dk2, dv2 = sdpAttentionBackward(go * 2, q, k, v, out, isCausal=True)
    assert torch.equal(dq2, dq * 2) and torch.equal(dk2, dk * 2) and torch.equal(dv2, dv * 2)
    colsum = dk.float().sum(dim=2).abs().max().item()
    assert colsum <= 2e-2 * N ** 0.5 * max(1.0, dk.float().abs().max().item()), colsum
    # one batch entry, one KV head (its four query heads) on the fp32 kernels
    sl = lambda t, h0, h1: t[1:2, h0:h1].float().contiguous()
    qf, kf, vf, gf = sl(q, 8, 12), sl(k, 2, 3), sl(v, 2, 3), sl(go, 8, 12)
    of = sdpAttention(qf, kf, vf, isCausal=True)
    rq, rk, rv = sdpAttentionBackward(gf, qf, kf, vf, of, isCausal=True)
    for got, ref in ((dq[1:2, 8:12], rq), (dk[1:2, 2:3], rk), (dv[1:2, 2:3], rv)):
        err = (got.float() - ref).abs().max().item() / max(1.0, ref.abs().max().item())
        assert err <= TOL["bf16"], err


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("kind", ["bool", "add", "keypad", "perhead"])
def test_backward_with_masks(dtype, kind):
    B, Hq, Hkv, L, S, D = 2, 4, 2, 19, 45, 64
    host, dev = make_inputs(4100, B, Hq, Hkv, L, S, D, dtype)
    rng = np.random.default_rng(3)
    if kind == "bool":
        m = rng.random((L, S)) < 0.7
        m[:, 0] = True
    elif kind == "add":
        m = oracle.round_to(rng.standard_normal((L, S)).astype(np.float32), dtype)[0]
    elif kind == "keypad":
        m = np.arange(S)[None, None, None, :] < np.array([S, 30])[:, None, None, None]   # [B,1,1,S]
    else:
        m = rng.random((Hq, L, S)) < 0.7                                                    # [Hq,L,S]
        m[..., 0] = True
    md = torch.from_numpy(np.ascontiguousarray(m)).cuda()
    if md.dtype != torch.bool:
        md = md.to(TORCH_DTYPE[dtype])
    check("mask-%s-%s" % (kind, dtype), host, dev, dtype, mask_h=m, mask_d=md, route="general")


@pytest.mark.parametrize("dtype,D", [("bf16", 128), ("f16", 64), ("f32", 128), ("f32", 64)])
@pytest.mark.parametrize("kind", ["bool", "add", "keypad", "perhead", "hiddenrow"])
def test_backward_mfma_with_masks(dtype, D, kind):
    """attnMasks the MFMA pair takes (contiguous keys, S a multiple of 4): Bool [L,S], additive [L,S], key padding
    [B,1,1,S], per-head [Hq,L,S]; and a mask with one fully hidden query row, whose dq is 0 and which adds nothing to dk / dv
    (the oracle, like the forward, has NaN there: that row is left out of the comparison)."""
    B, Hq, Hkv, L, S = 2, 4, 2, 70, 132
    host, dev = make_inputs(4500 + D, B, Hq, Hkv, L, S, D, dtype)
    rng = np.random.default_rng(4)
    if kind == "bool" or kind == "hiddenrow":
        m = rng.random((L, S)) < 0.7
        m[:, 0] = True
        if kind == "hiddenrow":
            m[5, :] = False
    elif kind == "add":
        m = oracle.round_to(rng.standard_normal((L, S)).astype(np.float32), dtype)[0]
    elif kind == "keypad":
        m = np.arange(S)[None, None, None, :] < np.array([S, 77])[:, None, None, None]
    else:
        m = rng.random((Hq, L, S)) < 0.7
        m[..., 0] = True
    md = torch.from_numpy(np.ascontiguousarray(m)).cuda()
    if md.dtype != torch.bool:
        md = md.to(TORCH_DTYPE[dtype])
    if kind != "hiddenrow":
        check("mfma-mask-%s-%s" % (kind, dtype), host, dev, dtype, mask_h=m, mask_d=md, route="prefill")
        return
    say("backward mfma hidden row", dtype, D)
    q, k, v = dev
    go_h, go = upstream(9, q.shape, dtype)
    rc, out = call("forward", q, k, v, mask=md)
    assert rc == 0
    out = torch.nan_to_num(out)   # the hidden row's forward output is NaN; the backward must not depend on it
    assert backward_route_of(q, k, v, out, go, False, md) == "prefill"
    rc, (dq, dk, dv) = backward_call(q, k, v, out, go, mask=md)
    assert rc == 0 and torch.all(dq[:, :, 5] == 0)
    keep = np.ones(L, bool)
    keep[5] = False
    eq, ek, ev = oracle.sdpa_backward_f32(host[0][:, :, keep], host[1], host[2], go_h[:, :, keep], mask=m[keep])
    assert grad_err(dq[:, :, torch.from_numpy(keep).cuda()], eq) <= TOL[dtype]
    assert grad_err(dk, ek) <= TOL[dtype] and grad_err(dv, ev) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_backward_bottom_right_causal_and_key_counts(dtype):
    """Bottom-right alignment with per-batch key counts: the oracle sees it as a Bool mask per batch entry; rows of
    dk / dv at or beyond the count are zero."""
    B, Hq, Hkv, L, S, D = 3, 4, 2, 12, 90, 64
    host, dev = make_inputs(4200, B, Hq, Hkv, L, S, D, dtype)
    lens = [90, 40, 13]
    kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
    m = np.zeros((B, 1, L, S), dtype=bool)
    for b in range(B):
        m[b, 0] = np.arange(S)[None, :] <= np.arange(L)[:, None] + lens[b] - L
        m[b, 0, :, lens[b]:] = False
    check("br-%s" % dtype, host, dev, dtype, causal=True, kv_lens=kv, align="bottom-right", oracle_mask=m)
    q, k, v = dev
    go = upstream(1, q.shape, dtype)[1]
    out = sdpAttention(q, k, v, isCausal=True, causalAlign="bottom-right", kvLens=kv)
    _, dk, dv = sdpAttentionBackward(go, q, k, v, out, isCausal=True, causalAlign="bottom-right", kvLens=kv)
    for b in range(B):
        assert torch.all(dk[b, :, lens[b]:] == 0) and torch.all(dv[b, :, lens[b]:] == 0)


@pytest.mark.parametrize("dtype,D", [("bf16", 128), ("f16", 64), ("f32", 128), ("f32", 64)])
@pytest.mark.parametrize("causal", [False, True])
def test_backward_mfma_per_batch_key_counts(dtype, D, causal):
    """kv_len on the MFMA pair: each batch entry against the oracle on its own key prefix (bottom-right causal when
    asked); an empty entry gets dq = 0; dk / dv beyond a count are zeros."""
    B, Hq, Hkv, L, S = 3, 8, 2, 70, 300
    host, dev = make_inputs(4400 + D, B, Hq, Hkv, L, S, D, dtype)
    lens = [300, 129, 0]
    kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
    q, k, v = dev
    go_h, go = upstream(5, q.shape, dtype)
    say("backward kv_len", dtype, D, causal)
    out = sdpAttention(q, k, v, isCausal=causal, causalAlign="bottom-right", kvLens=kv)
    assert backward_route_of(q, k, v, out, go, causal, None, None, kv, "bottom-right") == "prefill"
    rc, (dq, dk, dv) = backward_call(q, k, v, out, go, causal=causal, kv_lens=kv, align="bottom-right")
    assert rc == 0
    for b in range(B):
        n = lens[b]
        if n == 0:
            assert torch.all(dq[b] == 0) and torch.all(dk[b] == 0) and torch.all(dv[b] == 0)
            continue
        m = (np.arange(n)[None, :] <= np.arange(L)[:, None] + max(0, n - L)) if causal else None
        eq, ek, ev = oracle.sdpa_backward_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n],
                                              go_h[b:b + 1], mask=m)
        assert grad_err(dq[b:b + 1], eq) <= TOL[dtype], b
        assert grad_err(dk[b:b + 1, :, :n], ek) <= TOL[dtype], b
        assert grad_err(dv[b:b + 1, :, :n], ev) <= TOL[dtype], b
        assert torch.all(dk[b, :, n:] == 0) and torch.all(dv[b, :, n:] == 0)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("mode", ["causal", "full", "kvlen", "mask"])
def test_backward_split_query_stream(dtype, D, mode):
    """Matrix-core pairs with few key blocks and a long query stream (4 heads x 17 tiles per KV head): the dk/dv kernel
    deals the stream out to four workgroups per key block and a third kernel adds their fp32 partial sums.  The scratch
    the library asks for holds the partials (more than the 8 bytes per query row of the statistics)."""
    B, Hq, Hkv, L, S = 2, 8, 2, 520, 300
    host, dev = make_inputs(4700 + D, B, Hq, Hkv, L, S, D, dtype)
    q, k, v = dev
    go = upstream(9, q.shape, dtype)[1]
    out = sdpAttention(q, k, v, isCausal=(mode == "causal"))
    bp = build_backward_params(q, k, v, out, go, torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), mode == "causal")
    assert _capi.lib().ttsdpa_backward_workspace_bytes(ctypes.byref(bp)) >= B * Hq * L * 8 + 4 * 2 * B * Hkv * S * D * 4
    name = "split-%s-%s-%d" % (mode, dtype, D)
    if mode == "kvlen":
        lens = [300, 129]
        kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
        m = np.zeros((B, 1, L, S), dtype=bool)
        for b in range(B):
            m[b, 0] = np.arange(S)[None, :] <= np.arange(L)[:, None] + max(0, lens[b] - L)
            m[b, 0, :, lens[b]:] = False
        check(name, host, dev, dtype, causal=True, kv_lens=kv, align="bottom-right", oracle_mask=m, route="prefill")
        _, dk, dv = sdpAttentionBackward(go, q, k, v, sdpAttention(q, k, v, isCausal=True, causalAlign="bottom-right", kvLens=kv),
                                         isCausal=True, causalAlign="bottom-right", kvLens=kv)
        assert torch.all(dk[1, :, 129:] == 0) and torch.all(dv[1, :, 129:] == 0)
    elif mode == "mask":
        m = np.random.default_rng(6).random((Hq, L, S)) < 0.6
        m[..., 0] = True
        check(name, host, dev, dtype, mask_h=m, mask_d=torch.from_numpy(m).cuda(), route="prefill")
    else:
        check(name, host, dev, dtype, causal=(mode == "causal"), route="prefill")


@pytest.mark.parametrize("dtype,D", [("bf16", 128), ("f16", 64), ("f16", 128), ("bf16", 64), ("f32", 128), ("f32", 64)])
@pytest.mark.parametrize("mode", ["causal", "full", "br-kvlen", "mask", "hiddenrow"])
def test_backward_split_key_ranges(dtype, D, mode):
    """Matrix-core pairs with few query blocks and many keys: the dq kernel deals the key range of every 128-row
    query block out to several workgroups (here eight: 8 query blocks, 2100 keys) and a merge kernel brings their fp32
    partial sums to the common maximum.  The scratch the library asks for holds the partial records."""
    B, Hq, Hkv, L, S = 1, 4, 2, 200, 2100
    host, dev = make_inputs(4900 + D, B, Hq, Hkv, L, S, D, dtype)
    q, k, v = dev
    go = upstream(9, q.shape, dtype)[1]
    bp = build_backward_params(q, k, v, torch.empty_like(q), go, torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
                               mode == "causal")
    assert _capi.lib().ttsdpa_backward_workspace_bytes(ctypes.byref(bp)) >= B * Hq * L * 8 + 4 * B * Hq * L * (D + 2) * 4
    name = "ksplit-%s-%s-%d" % (mode, dtype, D)
    if mode == "br-kvlen":
        # one query chunk at the end of 1500 valid keys of 2100; the oracle sees the alignment and the count as a Bool mask
        n = 1500
        kv = torch.tensor([n], dtype=torch.int32, device="cuda")
        m = np.zeros((B, 1, L, S), dtype=bool)
        m[0, 0] = np.arange(S)[None, :] <= np.arange(L)[:, None] + (n - L)
        m[0, 0, :, n:] = False
        check(name, host, dev, dtype, causal=True, kv_lens=kv, align="bottom-right", oracle_mask=m, route="prefill")
    elif mode == "mask":
        m = np.random.default_rng(8).random((Hq, L, S)) < 0.5
        m[..., 7] = True
        check(name, host, dev, dtype, mask_h=m, mask_d=torch.from_numpy(m).cuda(), route="prefill")
    elif mode == "hiddenrow":
        # rows whose keys are all hidden in some splits (keys 0..599 only) and one hidden in every split: dq = 0 there
        m = np.random.default_rng(9).random((L, S)) < 0.5
        m[:, 7] = True
        m[10:20, 600:] = False
        m[5, :] = False
        md = torch.from_numpy(m).cuda()
        go_h, go = upstream(9, q.shape, dtype)
        rc, out = call("forward", q, k, v, mask=md)
        assert rc == 0
        out = torch.nan_to_num(out)
        rc, (dq, dk, dv) = backward_call(q, k, v, out, go, mask=md)
        assert rc == 0 and torch.all(dq[:, :, 5] == 0)
        keep = np.ones(L, bool)
        keep[5] = False
        eq, ek, ev = oracle.sdpa_backward_f32(host[0][:, :, keep], host[1], host[2], go_h[:, :, keep], mask=m[keep])
        assert grad_err(dq[:, :, torch.from_numpy(keep).cuda()], eq) <= TOL[dtype]
        assert grad_err(dk, ek) <= TOL[dtype] and grad_err(dv, ev) <= TOL[dtype]
    else:
        check(name, host, dev, dtype, causal=(mode == "causal"), route="prefill")


def test_backward_split_key_ranges_with_empty_pieces_and_entries():
    """More splits than some query blocks have tiles (causal: the first block sees 128 keys, i.e. four 32-key tiles, dealt
    out to eight workgroups), and a batch entry without keys (dq = 0 from the merge kernel, dk = dv = 0)."""
    B, Hq, Hkv, L, S, D = 2, 1, 1, 4200, 4200, 128
    dtype = "bf16"
    host, dev = make_inputs(5151, B, Hq, Hkv, L, S, D, dtype)
    q, k, v = dev
    go_h, go = upstream(3, q.shape, dtype)
    kv = torch.tensor([S, 0], dtype=torch.int32, device="cuda")
    rc, out = call("forward", q, k, v, causal=True, kv_lens=kv)
    assert rc == 0
    rc, (dq, dk, dv) = backward_call(q, k, v, out, go, True, None, None, kv)
    assert rc == 0
    assert torch.count_nonzero(dq[1]).item() == 0 and torch.count_nonzero(dk[1]).item() == 0 and torch.count_nonzero(dv[1]).item() == 0
    eq, ek, ev = oracle.sdpa_backward_f32(host[0][:1], host[1][:1], host[2][:1], go_h[:1], causal=True, nthreads=8)
    assert grad_err(dq[:1], eq) <= TOL[dtype] and grad_err(dk[:1], ek) <= TOL[dtype] and grad_err(dv[:1], ev) <= TOL[dtype]


def test_backward_strided_views_and_scale():
    """q/k/v as slices of one packed projection output, gradients into slices of one packed buffer."""
    B, H, N, D = 2, 4, 40, 64
    gen = torch.Generator(device="cuda").manual_seed(3)
    qkv = torch.randn(B, N, 3, H, D, device="cuda", generator=gen)
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))      # [B,H,N,D] views, row stride 3*H*D
    go = torch.randn(B, H, N, D, device="cuda", generator=gen)
    out = sdpAttention(q, k, v, isCausal=True, scale=0.2)
    dqkv = torch.full_like(qkv, float("nan"))
    grads = tuple(dqkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    rc, _ = backward_call(q, k, v, out, go, causal=True, scale=0.2, grads=grads)
    assert rc == 0 and torch.isfinite(dqkv).all()
    eq, ek, ev = oracle.sdpa_backward_f32(to_host_f32(q), to_host_f32(k), to_host_f32(v), to_host_f32(go), causal=True, scale=0.2)
    for got, exp in zip(grads, (eq, ek, ev)):
        assert grad_err(got, exp) <= TOL["f32"]


def test_backward_mfma_packed_projection_views():
    """bf16 q/k/v as slices of one packed QKV projection output [B, N, 3, H, D] and the gradients written into slices of
    one packed buffer: row strides of 3*H*D elements on the MFMA pair (head_dim 128, the direct-load kernels)."""
    B, H, N, D = 2, 4, 300, 128
    gen = torch.Generator(device="cuda").manual_seed(4)
    qkv = torch.randn(B, N, 3, H, D, device="cuda", generator=gen).bfloat16()
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    go = torch.randn(B, H, N, D, device="cuda", generator=gen).bfloat16()
    out = sdpAttention(q, k, v, isCausal=True)
    assert backward_route_of(q, k, v, out, go, True) == "prefill"
    dqkv = torch.full_like(qkv, float("nan"))
    grads = tuple(dqkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    rc, _ = backward_call(q, k, v, out, go, causal=True, grads=grads)
    assert rc == 0 and torch.isfinite(dqkv).all()
    eq, ek, ev = oracle.sdpa_backward_f32(to_host_f32(q), to_host_f32(k), to_host_f32(v), to_host_f32(go), causal=True)
    for got, exp in zip(grads, (eq, ek, ev)):
        assert grad_err(got, exp) <= TOL["bf16"]


def test_backward_validation_and_empty_shapes():
    q = torch.randn(1, 2, 4, 64, device="cuda")
    k = torch.randn(1, 2, 6, 64, device="cuda")
    v = torch.randn(1, 2, 6, 64, device="cuda")
    out = sdpAttention(q, k, v)
    go = torch.randn_like(q)
    rc, _ = backward_call(q, k, v, out, go, ws_bytes=8)      # scratch too small
    assert rc == _capi.ERR_WORKSPACE
    with pytest.raises(ValueError):
        sdpAttentionBackward(go[:, :1], q, k, v, out)
    with pytest.raises(TypeError):
        sdpAttentionBackward(go.half(), q, k, v, out)
    # no keys: dq = 0, nothing else to write; no queries: dk = dv = 0
    k0, v0 = k[:, :, :0], v[:, :, :0]
    dq, dk, dv = sdpAttentionBackward(go, q, k0, v0, sdpAttention(q, k0, v0))
    assert torch.all(dq == 0) and dk.numel() == 0
    q0 = q[:, :, :0]
    dq, dk, dv = sdpAttentionBackward(q0, q0, k, v, sdpAttention(q0, k, v))
    assert dq.numel() == 0 and torch.all(dk == 0) and torch.all(dv == 0)


def test_backward_matches_torch_autograd():
    """A second, independent check: torch's autograd through plain fp32 matmul / softmax / matmul on the same device."""
    B, Hq, Hkv, L, S, D = 2, 6, 2, 37, 53, 64
    gen = torch.Generator(device="cuda").manual_seed(9)
    q = torch.randn(B, Hq, L, D, device="cuda", generator=gen, requires_grad=True)
    k = torch.randn(B, Hkv, S, D, device="cuda", generator=gen, requires_grad=True)
    v = torch.randn(B, Hkv, S, D, device="cuda", generator=gen, requires_grad=True)
    go = torch.randn(B, Hq, L, D, device="cuda", generator=gen)
    G = Hq // Hkv
    s = (q @ k.repeat_interleave(G, 1).transpose(-1, -2)) / D ** 0.5
    s = s.masked_fill(~torch.ones(L, S, dtype=torch.bool, device="cuda").tril(), float("-inf"))
    ref = torch.softmax(s, -1) @ v.repeat_interleave(G, 1)
    ref.backward(go)
    out = sdpAttention(q.detach(), k.detach(), v.detach(), isCausal=True)
    dq, dk, dv = sdpAttentionBackward(go, q.detach(), k.detach(), v.detach(), out, isCausal=True)
    for got, exp in ((dq, q.grad), (dk, k.grad), (dv, v.grad)):
        assert (got - exp).abs().max().item() <= 1e-4 * max(1.0, exp.abs().max().item())
