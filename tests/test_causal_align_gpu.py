"""Bottom-right aligned causal masks (the L queries are the last L positions of the keys) on every kernel.

The reference's isCausal is top-left aligned only (src/Function/FuncNNLayer.h:241-247); what it computes for the
bottom-right case is its attnMask path with the Bool mask tril(ones(L,S), S-L) (src/Function/FuncNNLayer.h:249-260),
so that is what the oracle is given here."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, call, make_inputs, max_abs_err, route_of, to_host_f32

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def br_mask(L, S):
    """uint8 [L,S]: key j visible to query i iff j <= i + max(0, S - L)."""
    off = max(0, S - L)
    return (np.arange(S)[None, :] <= np.arange(L)[:, None] + off).astype(np.uint8)


CASES = [
    # B, Hq, Hkv, L, S, D, dtype, expected route
    (1, 4, 2, 256, 640, 128, "bf16", "prefill"),    # pipelined kernel, offset a multiple of the tile
    (2, 4, 2, 300, 777, 128, "f16", "prefill"),     # offset 477: the diagonal straddles 32-key halves
    (1, 8, 2, 257, 258, 128, "bf16", "prefill"),    # offset 1
    (1, 4, 4, 1024, 1100, 128, "bf16", "prefill"),  # several row tiles, mirrored pairing
    (1, 2, 2, 100, 333, 128, "bf16", "prefill"),    # the 4-wavefront kernel (L <= 128)
    (2, 4, 2, 200, 333, 64, "f16", "prefill"),      # head_dim 64
    (1, 2, 1, 130, 200, 256, "bf16", "prefill"),    # head_dim 256
    (1, 4, 2, 150, 400, 128, "f32", "prefill"),     # fp32 MFMA kernel
    (2, 2, 2, 77, 99, 64, "f32", "prefill"),
    (1, 2, 2, 70, 131, 96, "f32", "prefill"),       # a head size between the fp32 templates
    (1, 2, 2, 70, 131, 90, "f32", "general"),       # vector-ALU kernel
    (1, 2, 1, 40, 90, 80, "bf16", "prefill"),       # a head size between the templates: the head_dim-96 kernel
    (1, 2, 1, 40, 90, 84, "bf16", "general"),       # rows that are not whole 16-byte chunks
    (2, 8, 2, 4, 2048, 128, "bf16", "prefill"),     # 16 rows per KV head: 4 new tokens, packed heads on the MFMA kernel
    (2, 8, 2, 2, 2048, 128, "bf16", "decode"),      # 8 rows per KV head: the streaming kernel
    (1, 4, 4, 3, 1000, 128, "f16", "decode"),       # 3 rows per KV head
    (2, 8, 4, 5, 700, 64, "bf16", "prefill"),       # head_dim 64, 10 rows per KV head
    (2, 8, 4, 3, 700, 64, "bf16", "decode"),        # head_dim 64, 6 rows per KV head
    (1, 28, 4, 2, 5000, 128, "bf16", "prefill"),    # 7 heads per KV head, 14 rows: packed, keys split
    (1, 28, 4, 1, 5000, 128, "bf16", "decode"),     # 7 rows per KV head, split cache
    (1, 4, 2, 1, 512, 128, "bf16", "decode"),       # one new token sees every key
    (1, 4, 2, 300, 200, 128, "bf16", "prefill"),    # fewer keys than queries: offset 0, the top-left mask
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-%s" % c)
def test_bottom_right_against_oracle(case):
    B, Hq, Hkv, L, S, D, dtype, route = case
    say("bottom-right", case)
    host, dev = make_inputs(7000 + L + S, B, Hq, Hkv, L, S, D, dtype)
    exp = oracle.sdpa_f32(*host, mask=br_mask(L, S))
    assert route_of(*dev, causal=True, align="bottom-right") == route
    rc, out = call("forward", *dev, causal=True, align="bottom-right")
    assert rc == 0
    err = max_abs_err(out, exp)
    say("   max-abs-err", err)
    assert err <= TOL[dtype]
    rc, out2 = call("general", *dev, causal=True, align="bottom-right")   # the vector-ALU kernel agrees
    assert rc == 0 and max_abs_err(out2, exp) <= TOL[dtype]
    if S > L > 1:   # it is not the top-left mask
        rc, out3 = call("forward", *dev, causal=True)
        assert rc == 0 and not np.allclose(to_host_f32(out3), to_host_f32(out), atol=1e-3)


@pytest.mark.parametrize("dtype,B,Hq,Hkv,L,Smax,D,lens", [
    ("bf16", 4, 4, 2, 256, 1024, 128, [1024, 700, 256, 100]),   # pipelined prefill kernel; 100 < L: offset clamps to 0
    ("f16", 3, 8, 2, 4, 900, 128, [900, 333, 4]),                # decode kernel, 16 rows per KV head
    ("bf16", 2, 4, 4, 3, 600, 64, [5, 600]),                     # decode kernel, head_dim 64
    ("f32", 2, 4, 2, 50, 200, 96, [200, 77]),                    # vector-ALU kernel
])
def test_bottom_right_with_per_batch_key_counts(dtype, B, Hq, Hkv, L, Smax, D, lens):
    """A chunk of L new tokens per batch entry against caches filled to different lengths (the new rows included)."""
    say("bottom-right + kv_len", dtype, B, Hq, Hkv, L, Smax, D, lens)
    host, dev = make_inputs(8000 + L + Smax, B, Hq, Hkv, L, Smax, D, dtype)
    kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
    rc, out = call("forward", *dev, causal=True, align="bottom-right", kv_lens=kv)
    assert rc == 0
    for b in range(B):
        n = lens[b]
        exp = oracle.sdpa_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n], mask=br_mask(L, n))
        assert max_abs_err(out[b:b + 1], exp) <= TOL[dtype], b


def test_chunked_prefill_equals_one_pass():
    """Config 3's shape: the causal pass over 4096 tokens, and the same rows computed as four chunks of 1024 queries
    against the keys so far (bottom-right aligned), agree to the 16-bit bar; the first chunk is the top-left case."""
    from tinytorch_amd import sdpAttention
    B, Hq, Hkv, S, D, C = 2, 32, 8, 4096, 128, 1024
    gen = torch.Generator(device="cuda").manual_seed(11)
    q = torch.randn(B, Hq, S, D, device="cuda", generator=gen).bfloat16()
    k = torch.randn(B, Hkv, S, D, device="cuda", generator=gen).bfloat16()
    v = torch.randn(B, Hkv, S, D, device="cuda", generator=gen).bfloat16()
    full = sdpAttention(q, k, v, isCausal=True)
    for c in range(S // C):
        say("chunk", c)
        end = (c + 1) * C
        part = sdpAttention(q[:, :, c * C:end], k[:, :, :end], v[:, :, :end], isCausal=True, causalAlign="bottom-right")
        err = (part.float() - full[:, :, c * C:end].float()).abs().max().item()
        assert err <= TOL["bf16"], (c, err)
    torch.cuda.synchronize()


# ---- many query rows per KV head against a long cache: packed heads, split keys ----------------------------------------

MULTIROW_CASES = [
    # B, Hq, Hkv, L, S, D, dtype, causal (bottom-right)
    (2, 32, 8, 8, 4096, 128, "bf16", True),      # 32 rows per KV head: packed into one row tile, keys split
    (2, 32, 8, 8, 4096, 128, "f16", False),
    (1, 8, 2, 20, 1000, 64, "bf16", True),       # head_dim 64, ragged key count
    (1, 28, 4, 5, 3000, 128, "bf16", True),      # 7 heads per KV head: 35 rows
    (1, 64, 8, 40, 2100, 128, "f16", True),      # 320 packed rows: three row tiles per KV head
    (1, 4, 4, 17, 8192, 128, "bf16", True),      # one head per KV head: nothing to pack, keys split
    (16, 16, 8, 12, 700, 128, "bf16", False),    # enough (batch, head) pairs: packed, not split
    (2, 16, 4, 1, 3000, 128, "f32", False),      # fp32 decode step: packed heads and split keys on the fp32 MFMA kernel
    (1, 8, 2, 6, 2500, 64, "f32", True),
    (1, 4, 4, 3, 4100, 128, "f32", True),        # fp32, one head per KV head: keys split
]


@pytest.mark.parametrize("case", MULTIROW_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-c%d" % c)
def test_packed_heads_and_split_keys(case):
    """Short-L calls beyond the decode kernel's 16 rows: the G heads of a KV head share a row tile of the 4-wavefront
    kernel and the keys may be divided among workgroups (partials merged by the decode path's merge kernel).  Both are
    internal to the prefill route: the result is the oracle's, with and without scratch."""
    B, Hq, Hkv, L, S, D, dtype, causal = case
    say("multi-row", case)
    host, dev = make_inputs(7700 + L + S, B, Hq, Hkv, L, S, D, dtype)
    exp = oracle.sdpa_f32(*host, mask=br_mask(L, S)) if causal else oracle.sdpa_f32(*host)
    kw = dict(causal=causal, align="bottom-right")
    assert route_of(*dev, **kw) == "prefill"
    rc, out = call("forward", *dev, **kw)    # with the scratch ttsdpa_workspace_bytes asks for
    assert rc == 0
    assert max_abs_err(out, exp) <= TOL[dtype]
    rc, out2 = call("prefill", *dev, **kw)   # no scratch: no split
    assert rc == 0 and max_abs_err(out2, exp) <= TOL[dtype]
    # per-batch key counts on the same path
    lens = [S - 37 * b for b in range(B)]
    kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
    rc, out3 = call("forward", *dev, kv_lens=kv, **kw)
    assert rc == 0
    for b in (0, B - 1):
        n = lens[b]
        e = oracle.sdpa_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n],
                            mask=br_mask(L, n) if causal else None)
        assert max_abs_err(out3[b:b + 1], e) <= TOL[dtype], b


def test_split_keys_need_scratch_only_when_asked():
    import ctypes
    from tinytorch_amd import _capi, build_params
    host, dev = make_inputs(1, 1, 32, 8, 8, 8192, 128, "bf16")
    out = torch.empty_like(dev[0])
    p = build_params(*dev, out, True, causalAlign="bottom-right")
    need = _capi.lib().ttsdpa_workspace_bytes(ctypes.byref(p))
    assert need > 0 and need % 4 == 0           # one (batch) x 8 KV heads: the keys are split
    big = make_inputs(2, 64, 32, 8, 8, 1024, 128, "bf16")[1]
    p2 = build_params(*big, torch.empty_like(big[0]), True, causalAlign="bottom-right")
    assert _capi.lib().ttsdpa_workspace_bytes(ctypes.byref(p2)) == 0   # 512 pairs fill the chip unsplit
