"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on identical seeded inputs.

Bars (north-star statement): max-abs-error <= 1e-4 for fp32, <= 2e-2 for fp16/bf16 (fp32 accumulation; the oracle is
the reference's fp32 CPU path applied to the inputs rounded to the 16-bit type)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import golden_names, load_golden
from gpu_util import TOL, call, make_inputs, max_abs_err, route_of, to_device, to_host_f32

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


# ---- fixtures written from the compiled reference ---------------------------------------------------------------

@pytest.mark.parametrize("name", golden_names())
def test_golden_fp32(name):
    g = load_golden(name)
    say("golden fp32", name)
    q, k, v = [torch.from_numpy(g[x]).cuda() for x in ("q", "k", "v")]
    mask = None
    if g["mask"] is not None:
        mask = torch.from_numpy(g["mask"]).cuda()
        mask = mask.bool() if g["mask"].dtype == np.uint8 else mask
    rc, out = call("forward", q, k, v, causal=g["causal"], mask=mask, scale=g["scale"])
    assert rc == 0
    y, exp = to_host_f32(out), g["out"]
    assert np.array_equal(np.isnan(y), np.isnan(exp))  # rows with every key hidden are NaN on both sides
    ok = ~np.isnan(exp)
    assert np.abs(y[ok] - exp[ok]).max() <= TOL["f32"]


@pytest.mark.parametrize("name,dtype", [("bf16_inputs_causal", "bf16"), ("f16_inputs_causal", "f16"),
                                        ("decode_l1_s64", "bf16"), ("decode_l1_s300_scale", "f16"),
                                        ("gqa_hq8_hkv2", "bf16"), ("boolmask_l9_s12", "bf16"),
                                        ("floatmask_l9_s12", "f16")])
def test_golden_16bit(name, dtype):
    g = load_golden(name)
    say("golden", dtype, name)
    host, dev = [], []
    for x in ("q", "k", "v"):
        vals, bits = oracle.round_to(g[x], dtype)
        host.append(vals)
        dev.append(to_device(vals, bits, dtype))
    mask_h, mask_d = g["mask"], None
    if mask_h is not None:
        if mask_h.dtype == np.uint8:
            mask_d = torch.from_numpy(mask_h).cuda().bool()
        else:
            mv, mb = oracle.round_to(mask_h, dtype)
            mask_h, mask_d = mv, to_device(mv, mb, dtype)
    exp = oracle.sdpa_f32(*host, causal=g["causal"], scale=g["scale"], mask=mask_h)
    rc, out = call("forward", *dev, causal=g["causal"], mask=mask_d, scale=g["scale"])
    assert rc == 0
    assert max_abs_err(out, exp) <= TOL[dtype]


# ---- config 1 exactly --------------------------------------------------------------------------------------------

def test_config1_fp32_causal():
    host, dev = make_inputs(0x5EED0001, 1, 4, 4, 128, 128, 64, "f32")
    g = load_golden("c1_f32_causal")
    assert np.array_equal(host[0], g["q"])  # the fixture holds these very inputs
    rc, out = call("forward", *dev, causal=True)
    assert rc == 0
    err = max_abs_err(out, g["out"])
    say("config1 fp32 max-abs-err vs reference output:", err)
    assert err <= 1e-4


# ---- prefill kernel ------------------------------------------------------------------------------------------------

PREFILL_CASES = [
    # B, Hq, Hkv, L, S, D, dtype, causal, mul
    (1, 4, 4, 512, 512, 128, "f16", True, 0.5),     # config 2, scaled down
    (1, 8, 2, 1024, 1024, 128, "bf16", True, 1.0),  # config 3, scaled down
    (1, 7, 1, 768, 768, 128, "bf16", True, 1.0),    # config 5's 7-heads-per-KV-head grouping
    (2, 4, 2, 256, 256, 128, "bf16", False, 1.0),
    (1, 2, 2, 128, 128, 128, "f16", True, 1.0),
    (1, 2, 1, 100, 100, 128, "bf16", True, 1.0),    # ragged: not a multiple of any tile
    (1, 2, 2, 130, 257, 128, "bf16", False, 1.0),
    (1, 2, 2, 200, 77, 128, "f16", True, 1.0),      # L > S, top-left causal
    (1, 2, 2, 77, 200, 128, "bf16", True, 1.0),     # L < S
    (1, 3, 3, 33, 64, 128, "bf16", False, 1.0),
    (1, 4, 2, 300, 300, 64, "bf16", True, 1.0),     # head_dim 64
    (2, 2, 2, 129, 65, 64, "f16", False, 1.0),
    (1, 2, 2, 16, 16, 128, "bf16", True, 1.0),
    (8, 16, 8, 192, 192, 128, "bf16", True, 1.0),   # (batch x kv heads) multiple of 8: the XCD-aware order
]


@pytest.mark.parametrize("case", PREFILL_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-c%d" % c[:8])
def test_prefill_against_oracle(case):
    B, Hq, Hkv, L, S, D, dtype, causal, mul = case
    say("prefill", case)
    host, dev = make_inputs(1000 + L + S, B, Hq, Hkv, L, S, D, dtype, mul)
    exp = oracle.sdpa_f32(*host, causal=causal)
    rc, out = call("prefill", *dev, causal=causal)
    assert rc == 0
    err = max_abs_err(out, exp)
    say("   max-abs-err", err)
    assert err <= TOL[dtype]
    assert route_of(*dev, causal=causal) in ("prefill", "decode")
    rc, out2 = call("forward", *dev, causal=causal)
    assert rc == 0 and max_abs_err(out2, exp) <= TOL[dtype]


@pytest.mark.parametrize("entry,shape", [("prefill", (1, 4, 2, 512, 512, 128)), ("prefill", (1, 2, 2, 200, 200, 64)),
                                         ("decode", (2, 8, 2, 1, 2048, 128))])
def test_large_score_range(entry, shape):
    """Inputs scaled so that scores spread over hundreds of units: the running maximum has to follow every tile
    (a maximum taken over only part of a row's keys would overflow the exponentials)."""
    B, Hq, Hkv, L, S, D = shape
    host, dev = make_inputs(4242, B, Hq, Hkv, L, S, D, "bf16", mul=6.0)
    causal = entry == "prefill"
    exp = oracle.sdpa_f32(*host, causal=causal)
    rc, out = call(entry, *dev, causal=causal)
    assert rc == 0
    # values are 6x larger: the 2e-2 bar is relative to unit-variance inputs, scale it with the value range
    assert max_abs_err(out, exp) <= 6.0 * TOL["bf16"]


def test_prefill_custom_scale_and_strided_views():
    B, Hq, Hkv, L, S, D = 2, 4, 2, 160, 160, 128
    host, dev = make_inputs(77, B, Hq, Hkv, L, S, D, "bf16")
    exp = oracle.sdpa_f32(*host, causal=True, scale=0.03)
    # q arrives as a transposed view of a [B, L, H, D] buffer; k/v as the first S rows of a longer cache
    qbuf = dev[0].permute(0, 2, 1, 3).contiguous()
    qv = qbuf.permute(0, 2, 1, 3)
    assert not qv.is_contiguous()
    cache_k = torch.zeros(B, Hkv, S + 96, D, dtype=dev[1].dtype, device="cuda")
    cache_v = torch.zeros_like(cache_k)
    cache_k[:, :, :S] = dev[1]
    cache_v[:, :, :S] = dev[2]
    rc, out = call("prefill", qv, cache_k[:, :, :S], cache_v[:, :, :S], causal=True, scale=0.03)
    assert rc == 0
    assert max_abs_err(out, exp) <= TOL["bf16"]


def test_gqa_equals_repeated_kv_bitwise():
    """kv head = q head / G inside the kernel must be the same arithmetic as feeding repeat-interleaved K/V
    (what the reference does, src/Operation/OpTransformCpu.h:399-442)."""
    host, dev = make_inputs(5, 1, 8, 2, 384, 384, 128, "bf16")
    rc, a = call("prefill", *dev, causal=True)
    kr = dev[1].repeat_interleave(4, dim=1)
    vr = dev[2].repeat_interleave(4, dim=1)
    rc2, b = call("prefill", dev[0], kr, vr, causal=True)
    assert rc == 0 and rc2 == 0
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


# ---- decode kernel -------------------------------------------------------------------------------------------------

DECODE_CASES = [
    # B, Hq, Hkv, L, S, dtype
    (4, 32, 8, 1, 2048, "bf16"),   # config 4, scaled down (several splits)
    (2, 8, 2, 1, 1, "bf16"),
    (2, 8, 2, 1, 31, "bf16"),
    (2, 8, 2, 1, 32, "f16"),
    (2, 8, 2, 1, 33, "bf16"),
    (1, 4, 4, 1, 255, "bf16"),     # one query head per KV head
    (1, 8, 2, 1, 1000, "f16"),
    (3, 28, 4, 1, 777, "bf16"),    # 7 heads per KV head
    (1, 16, 2, 1, 4100, "bf16"),   # 8 per KV head, ragged tail
    (1, 16, 1, 1, 513, "bf16"),    # 16 per KV head
    (2, 4, 1, 4, 640, "bf16"),     # 4 query rows x 4 heads = 16 rows (multi-token decode)
    (2, 6, 2, 2, 300, "f16"),      # 2 rows x 3 heads
    (1, 32, 8, 1, 16384, "bf16"),  # long cache, many splits
]


@pytest.mark.parametrize("case", DECODE_CASES, ids=lambda c: "B%dH%dk%dL%dS%d-%s" % c)
def test_decode_against_oracle(case):
    B, Hq, Hkv, L, S, dtype = case
    say("decode", case)
    host, dev = make_inputs(2000 + S, B, Hq, Hkv, L, S, 128, dtype)
    exp = oracle.sdpa_f32(*host, causal=False)
    rc, out = call("decode", *dev)
    assert rc == 0
    err = max_abs_err(out, exp)
    say("   max-abs-err", err)
    assert err <= TOL[dtype]


@pytest.mark.parametrize("D", [8, 40, 56, 72, 80, 96, 112, 120])
@pytest.mark.parametrize("shape", [(4, 32, 8, 1, 2048, "bf16"), (2, 8, 2, 1, 33, "f16"), (1, 16, 1, 1, 513, "bf16"),
                                   (2, 4, 1, 4, 640, "f16"), (1, 32, 8, 1, 9000, "bf16")],
                         ids=lambda c: "B%dH%dk%dL%dS%d-%s" % c)
def test_decode_head_sizes_between_the_kernels(D, shape):
    # any multiple of 8 up to 128 on the streaming kernel for 64 or 128 (zero columns); views of wider rows whose other
    # columns hold NaN (inputs) or a sentinel (output), so that nothing beyond head_dim is read into the result or written
    B, Hq, Hkv, L, S, dtype = shape
    say("decode, padded head_dim", D, shape)
    host, dev = make_inputs(2300 + S + D, B, Hq, Hkv, L, S, D, dtype)
    assert route_of(*dev) == "decode"
    exp = oracle.sdpa_f32(*host, causal=False)
    rc, out = call("forward", *dev)
    assert rc == 0 and max_abs_err(out, exp) <= TOL[dtype]
    wide = []
    for t in dev:
        w = torch.full(t.shape[:-1] + (128,), float("nan"), dtype=t.dtype, device="cuda")
        w[..., :D] = t
        wide.append(w[..., :D])
    outw = torch.full((B, Hq, L, 128), 7.0, dtype=dev[0].dtype, device="cuda")
    rc, _ = call("decode", *wide, out=outw[..., :D])
    assert rc == 0 and torch.equal(outw[..., :D], out) and bool((outw[..., D:] == 7.0).all())
    # per-batch key counts and the bottom-right causal rows of a multi-token step
    if S >= 513:
        lens = np.array([S - 5 * b for b in range(B)], np.int32)
        rc, out = call("forward", *dev, causal=L > 1, align="bottom-right", kv_lens=torch.from_numpy(lens).cuda())
        assert rc == 0
        for b in range(B):
            n = int(lens[b])
            m = np.tril(np.ones((L, n), np.uint8), n - L)
            e = oracle.sdpa_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n], mask=m)
            assert max_abs_err(out[b:b + 1], e) <= TOL[dtype]


def test_decode_cache_view_and_key_permutation():
    B, Hq, Hkv, S, D = 4, 8, 2, 1500, 128
    host, dev = make_inputs(31, B, Hq, Hkv, 1, S, D, "bf16")
    exp = oracle.sdpa_f32(*host)
    cache_k = torch.zeros(B, Hkv, 2048, D, dtype=torch.bfloat16, device="cuda")
    cache_v = torch.zeros_like(cache_k)
    cache_k[:, :, :S] = dev[1]
    cache_v[:, :, :S] = dev[2]
    rc, out = call("forward", dev[0], cache_k[:, :, :S], cache_v[:, :, :S])
    assert rc == 0 and max_abs_err(out, exp) <= TOL["bf16"]
    # attention without a mask does not care about the order of the cache entries
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(1)).cuda()
    rc, outp = call("forward", dev[0], dev[1][:, :, perm].contiguous(), dev[2][:, :, perm].contiguous())
    assert rc == 0
    assert np.abs(to_host_f32(out) - to_host_f32(outp)).max() <= 1e-2


def test_all_routes_agree():
    """The three kernels are three schedules of the same function."""
    host, dev = make_inputs(41, 2, 8, 2, 4, 512, 128, "bf16")
    exp = oracle.sdpa_f32(*host)
    outs = {}
    for entry in ("general", "prefill", "decode"):
        rc, o = call(entry, *dev)
        assert rc == 0, entry
        outs[entry] = o
        assert max_abs_err(o, exp) <= TOL["bf16"], entry
    a, b, c = [to_host_f32(outs[e]) for e in ("general", "prefill", "decode")]
    assert np.abs(a - b).max() <= 1e-2 and np.abs(a - c).max() <= 1e-2


# ---- general kernel ------------------------------------------------------------------------------------------------

GENERAL_CASES = [
    (1, 2, 2, 70, 70, 64, "f32", True), (2, 4, 2, 33, 90, 96, "f32", False), (1, 2, 1, 65, 65, 256, "f32", True),
    (1, 3, 3, 5, 7, 20, "f32", False), (1, 2, 2, 64, 64, 96, "bf16", True), (1, 2, 2, 40, 50, 32, "f16", False),
    (1, 1, 1, 1, 1, 4, "f32", True), (1, 2, 2, 130, 64, 6, "f32", True),
]


@pytest.mark.parametrize("case", GENERAL_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-c%d" % c)
def test_general_against_oracle(case):
    B, Hq, Hkv, L, S, D, dtype, causal = case
    say("general", case)
    host, dev = make_inputs(3000 + D, B, Hq, Hkv, L, S, D, dtype)
    exp = oracle.sdpa_f32(*host, causal=causal)
    rc, out = call("general", *dev, causal=causal)
    assert rc == 0
    assert max_abs_err(out, exp) <= TOL[dtype]
    if dtype == "f32":
        assert route_of(*dev, causal=causal) == ("prefill" if D % 4 == 0 and D <= 128 else "general")


def test_general_masks_large():
    B, Hq, Hkv, L, S, D = 2, 4, 2, 150, 170, 128
    host, dev = make_inputs(55, B, Hq, Hkv, L, S, D, "bf16")
    rng = np.random.RandomState(2)
    bm = (rng.rand(L, S) > 0.5).astype(np.uint8)
    bm[:, 3] = 1
    exp = oracle.sdpa_f32(*host, mask=bm)
    rc, out = call("forward", *dev, mask=torch.from_numpy(bm).cuda().bool())
    assert rc == 0 and max_abs_err(out, exp) <= TOL["bf16"]
    fm_v, fm_b = oracle.round_to(oracle.randn(56, 9, (L, S)), "bf16")
    exp = oracle.sdpa_f32(*host, mask=fm_v)
    rc, out = call("forward", *dev, mask=to_device(fm_v, fm_b, "bf16"))
    assert rc == 0 and max_abs_err(out, exp) <= TOL["bf16"]


@pytest.mark.parametrize("mshape", [(1, 1, 1, 170), (2, 1, 1, 170), (2, 1, 70, 170), (2, 4, 70, 170), (4, 70, 1), (170,)])
@pytest.mark.parametrize("kind,dtype", [("bool", "bf16"), ("float", "f16"), ("float", "f32")])
def test_broadcast_mask_shapes(mshape, kind, dtype):
    # attnMask of any shape that broadcasts to [B,H,L,S] (reference src/Function/FuncNNLayer.h:249-260)
    B, Hq, Hkv, L, S, D = 2, 4, 2, 70, 170, 64
    host, dev = make_inputs(57, B, Hq, Hkv, L, S, D, dtype)
    if kind == "bool":
        m = (np.random.RandomState(len(mshape)).rand(*mshape) > 0.5).astype(np.uint8)
        m[..., 0] = 1  # no row without a visible key
        md = torch.from_numpy(m).cuda().bool()
    else:
        m, bits = oracle.round_to(oracle.randn(58, 9, mshape), dtype)
        md = to_device(m, bits, dtype)
    exp = oracle.sdpa_f32(*host, mask=m)
    rc, out = call("forward", *dev, mask=md)
    assert rc == 0 and max_abs_err(out, exp) <= TOL[dtype]


def test_mask_views_with_strides():
    # the mask is described by element strides: an expanded view (stride 0) and a sliced view (row and key strides
    # that are not dense) give the result of their materialised copies
    B, Hq, Hkv, L, S, D = 2, 4, 4, 33, 50, 32
    host, dev = make_inputs(59, B, Hq, Hkv, L, S, D, "f32")
    big = oracle.randn(60, 9, (B, 2 * L, 2 * S))
    view = torch.from_numpy(big).cuda()[:, ::2, 1::2].unsqueeze(1)  # [B,1,L,S], strides (4LS, -, 4S, 2)
    assert not view.is_contiguous()
    exp = oracle.sdpa_f32(*host, mask=np.ascontiguousarray(big[:, None, ::2, 1::2]))
    rc, out = call("forward", *dev, mask=view)
    assert rc == 0 and max_abs_err(out, exp) <= TOL["f32"]
    keypad = torch.ones(B, 1, 1, S, dtype=torch.bool, device="cuda")
    keypad[0, ..., 20:] = False
    rc, out2 = call("forward", *dev, mask=keypad.expand(B, Hq, L, S))
    exp2 = oracle.sdpa_f32(*host, mask=keypad.cpu().numpy().astype(np.uint8))
    assert rc == 0 and max_abs_err(out2, exp2) <= TOL["f32"]
    # hidden keys do not influence the result at all: batch 0 equals attention over its first 20 keys
    rc, out3 = call("forward", dev[0][:1], dev[1][:1, :, :20], dev[2][:1, :, :20])
    assert rc == 0 and torch.allclose(out2[:1], out3, atol=1e-5)


def test_empty_and_degenerate_shapes():
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device="cuda")
    rc, out = call("forward", z(2, 4, 0, 128), z(2, 4, 16, 128), z(2, 4, 16, 128))
    assert rc == 0 and out.numel() == 0
    rc, out = call("forward", z(0, 4, 8, 128), z(0, 4, 16, 128), z(0, 4, 16, 128))
    assert rc == 0 and out.numel() == 0
    # S == 0: the reference's empty contraction gives zeros
    out = torch.full((2, 4, 8, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    rc, out = call("forward", z(2, 4, 8, 128) + 1, z(2, 4, 0, 128), z(2, 4, 0, 128), out=out)
    assert rc == 0 and float(out.float().abs().max()) == 0.0


def test_host_wrapper_matches_capi():
    from tinytorch_amd import sdpAttention
    host, dev = make_inputs(61, 1, 8, 2, 256, 256, 128, "bf16")
    y = sdpAttention(*dev, isCausal=True)
    rc, out = call("forward", *dev, causal=True)
    assert rc == 0 and torch.equal(y.view(torch.int16), out.view(torch.int16))
    hostd, devd = make_inputs(62, 2, 8, 2, 1, 3000, 128, "bf16")
    y = sdpAttention(*devd)
    assert max_abs_err(y, oracle.sdpa_f32(*hostd)) <= TOL["bf16"]


# ---- KV cache: append in place + per-batch key counts (what a token-by-token caller of the reference would get from
# growing K/V with op::concat and calling sdpAttention on the grown tensors) -------------------------------------------

def _cache_case(dtype, B, Hq, Hkv, D, Smax, seed):
    kfull = oracle.randn(seed, 1, (B, Hkv, Smax, D))
    vfull = oracle.randn(seed, 2, (B, Hkv, Smax, D))
    kv, kb = oracle.round_to(kfull, dtype)
    vv, vb = oracle.round_to(vfull, dtype)
    return kv, vv, to_device(kv, kb, dtype), to_device(vv, vb, dtype)


@pytest.mark.parametrize("dtype,B,Hq,Hkv,D,Smax,L", [
    ("bf16", 3, 8, 2, 128, 700, 1),    # decode route, one row per head
    ("f16", 2, 8, 8, 128, 300, 1),
    ("bf16", 2, 8, 2, 128, 520, 3),    # three new tokens per step (12 rows per KV head)
    ("f32", 2, 4, 2, 64, 90, 1),       # general route
    ("bf16", 2, 4, 4, 64, 130, 2),     # general route, 16-bit, head_dim 64
])
def test_kv_cache_generation_matches_concat(dtype, B, Hq, Hkv, D, Smax, L):
    from tinytorch_amd import kvCacheAppend, sdpAttention
    kh, vh, kd, vd = _cache_case(dtype, B, Hq, Hkv, D, Smax, 70 + Smax)
    kc = torch.zeros_like(kd)
    vc = torch.zeros_like(vd)
    # prompts of different lengths, appended in one call per batch entry count: position 0, Lnew = the longest prompt,
    # then the shorter entries simply report a smaller length (their extra rows are overwritten later)
    lens = np.array([(37 * (b + 1)) % (Smax // 2) + 5 for b in range(B)], np.int32)
    pmax = int(lens.max())
    kvCacheAppend(kc, vc, kd[:, :, :pmax], vd[:, :, :pmax], 0)
    steps = 4
    for step in range(steps):
        pos = torch.from_numpy(lens).cuda()
        # the new tokens of batch b are rows lens[b] .. lens[b]+L-1 of the full tensors: gather them per batch entry
        knew = torch.stack([kd[b, :, lens[b]:lens[b] + L] for b in range(B)])
        vnew = torch.stack([vd[b, :, lens[b]:lens[b] + L] for b in range(B)])
        kvCacheAppend(kc, vc, knew, vnew, pos)
        lens = lens + L
        qh, qb = oracle.round_to(oracle.randn(900 + step, 0, (B, Hq, L, D)), dtype)
        q = to_device(qh, qb, dtype)
        out = sdpAttention(q, kc, vc, kvLens=torch.from_numpy(lens).cuda())
        torch.cuda.synchronize()
        for b in range(B):
            exp = oracle.sdpa_f32(qh[b:b + 1], kh[b:b + 1, :, :lens[b]], vh[b:b + 1, :, :lens[b]])
            assert max_abs_err(out[b:b + 1], exp) <= TOL[dtype], (step, b)
    # the caches hold exactly the rows of the full tensors up to each length
    for b in range(B):
        assert torch.equal(kc[b, :, :lens[b]], kd[b, :, :lens[b]]) and torch.equal(vc[b, :, :lens[b]], vd[b, :, :lens[b]])


def test_kv_len_edge_cases():
    from tinytorch_amd import kvCacheAppend, sdpAttention
    B, Hq, Hkv, D, Smax = 3, 4, 2, 128, 600
    kh, vh, kd, vd = _cache_case("bf16", B, Hq, Hkv, D, Smax, 77)
    qh, qb = oracle.round_to(oracle.randn(78, 0, (B, Hq, 1, D)), "bf16")
    q = to_device(qh, qb, "bf16")
    lens = torch.tensor([0, 1, 9999], dtype=torch.int32, device="cuda")  # empty, one key, more than the cache holds
    for route_q, tol in ((q, TOL["bf16"]), (q.float(), TOL["f32"])):   # decode route, then general route (fp32)
        k, v = (kd, vd) if route_q.dtype == torch.bfloat16 else (kd.float(), vd.float())
        out = sdpAttention(route_q, k, v, kvLens=lens)
        assert torch.count_nonzero(out[0]) == 0                       # no keys: zeros, the reference's empty contraction
        assert max_abs_err(out[1:2], np.repeat(vh[1:2, :, 0:1, :], Hq // Hkv, axis=1)) <= tol  # one key: its value row
        assert max_abs_err(out[2:3], oracle.sdpa_f32(qh[2:3], kh[2:3], vh[2:3])) <= tol
    # rows that do not fit the cache are dropped, everything else is untouched
    kc, vc = torch.zeros_like(kd), torch.zeros_like(vd)
    kvCacheAppend(kc, vc, kd[:, :, :4], vd[:, :, :4], torch.tensor([Smax - 2, 10, Smax + 5], dtype=torch.int32, device="cuda"))
    assert torch.equal(kc[0, :, Smax - 2:], kd[0, :, :2]) and torch.count_nonzero(kc[0, :, :Smax - 2]) == 0
    assert torch.equal(kc[1, :, 10:14], kd[1, :, :4]) and torch.count_nonzero(kc[2]) == 0
    # strided cache views and rows narrower than 16 bytes
    big = torch.zeros(2, 2, 50, 2 * 20, dtype=torch.float16, device="cuda")
    kc2, vc2 = big[..., :20], big[..., 20:]
    kn = torch.randn(2, 2, 3, 20, device="cuda").half()
    vn = torch.randn(2, 2, 3, 20, device="cuda").half()
    kvCacheAppend(kc2, vc2, kn, vn, 7)
    assert torch.equal(kc2[:, :, 7:10], kn) and torch.equal(vc2[:, :, 7:10], vn) and torch.count_nonzero(big[:, :, :7]) == 0
    kc3 = torch.zeros(1, 1, 9, 3, dtype=torch.bfloat16, device="cuda")
    vc3 = torch.zeros_like(kc3)
    kn3 = torch.randn(1, 1, 2, 3, device="cuda").bfloat16()
    kvCacheAppend(kc3, vc3, kn3, kn3, 5)
    assert torch.equal(kc3[:, :, 5:7], kn3) and torch.equal(vc3[:, :, 5:7], kn3)


# ---- attnMask on the pipelined MFMA kernel (head_dim 128, more than 128 query rows) -------------------------------------

@pytest.mark.parametrize("mshape,kind", [((2, 1, 1, 600), "bool"), ((300, 600), "bool"), ((2, 8, 300, 600), "float"),
                                         ((8, 1, 600), "float"), ((2, 1, 300, 1), "float")])
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_masks_on_the_mfma_route(mshape, kind, dtype):
    B, Hq, Hkv, L, S, D = 2, 8, 2, 300, 600, 128
    host, dev = make_inputs(91, B, Hq, Hkv, L, S, D, dtype)
    if kind == "bool":
        m = (np.random.RandomState(len(mshape)).rand(*mshape) > 0.5).astype(np.uint8)
        m[..., 5] = 1
        md = torch.from_numpy(m).cuda().bool()
    else:
        m, bits = oracle.round_to(oracle.randn(92, 9, mshape, 2.0), dtype)
        md = to_device(m, bits, dtype)
    assert route_of(*dev, mask=md) == "prefill"
    exp = oracle.sdpa_f32(*host, mask=m)
    rc, out = call("forward", *dev, mask=md)
    assert rc == 0 and max_abs_err(out, exp) <= TOL[dtype]
    rc, out2 = call("general", *dev, mask=md)   # the vector-ALU kernel agrees
    assert rc == 0 and max_abs_err(out2, exp) <= TOL[dtype]


def test_fully_hidden_rows_on_the_mfma_route():
    # rows whose mask hides every key are NaN in the reference (0 * inf); rows hidden only partly are not affected
    B, Hq, Hkv, L, S, D = 1, 4, 2, 260, 200, 128
    host, dev = make_inputs(93, B, Hq, Hkv, L, S, D, "bf16")
    m = np.ones((L, S), np.uint8)
    m[7] = 0
    m[200:230] = 0
    m[100, 50:] = 0
    md = torch.from_numpy(m).cuda().bool()
    assert route_of(*dev, mask=md) == "prefill"
    exp = oracle.sdpa_f32(*host, mask=m)
    rc, out = call("forward", *dev, mask=md)
    y = to_host_f32(out)
    assert rc == 0 and np.array_equal(np.isnan(y), np.isnan(exp)) and np.isnan(exp[0, :, 7]).all() and not np.isnan(exp[0, :, 100]).any()
    ok = ~np.isnan(exp)
    assert np.abs(y[ok] - exp[ok]).max() <= TOL["bf16"]


@pytest.mark.parametrize("D", [32, 96, 256])
@pytest.mark.parametrize("dtype,causal", [("bf16", True), ("f16", False)])
def test_other_head_sizes_on_the_mfma_route(D, dtype, causal):
    B, Hq, Hkv, L, S = 2, 6, 2, 333, 333 if causal else 411
    host, dev = make_inputs(95 + D, B, Hq, Hkv, L, S, D, dtype, 0.7)
    assert route_of(*dev, causal=causal) == "prefill"
    exp = oracle.sdpa_f32(*host, causal=causal)
    rc, out = call("forward", *dev, causal=causal)
    assert rc == 0 and max_abs_err(out, exp) <= TOL[dtype]


@pytest.mark.parametrize("D", [8, 24, 40, 56, 72, 80, 112, 120, 136, 160, 192, 200, 248])
@pytest.mark.parametrize("dtype,causal", [("bf16", True), ("f16", False)])
def test_head_sizes_between_the_mfma_kernels(D, dtype, causal):
    # any multiple of 8 up to 256 runs on the matrix-core kernel of the next size up (the reference takes any head size)
    B, Hq, Hkv, L, S = 2, 6, 2, 200, 200 if causal else 330
    say("padded head_dim", (D, dtype, causal))
    host, dev = make_inputs(195 + D, B, Hq, Hkv, L, S, D, dtype, 0.7)
    assert route_of(*dev, causal=causal) == "prefill"
    exp = oracle.sdpa_f32(*host, causal=causal)
    rc, out = call("forward", *dev, causal=causal)
    assert rc == 0 and max_abs_err(out, exp) <= TOL[dtype]


@pytest.mark.parametrize("D", [4, 20, 36, 60, 68, 96, 100, 124])
@pytest.mark.parametrize("causal", [True, False])
def test_fp32_head_sizes_between_the_mfma_kernels(D, causal):
    # fp32 tensors: any multiple of 4 up to 128 runs on the fp32 matrix-core kernel for 64 or 128 (zero columns)
    B, Hq, Hkv, L, S = 2, 4, 2, 150, 150 if causal else 233
    say("padded head_dim, fp32", (D, causal))
    host, dev = make_inputs(295 + D, B, Hq, Hkv, L, S, D, "f32", 0.7)
    assert route_of(*dev, causal=causal) == "prefill"
    exp = oracle.sdpa_f32(*host, causal=causal)
    rc, out = call("forward", *dev, causal=causal)
    assert rc == 0 and max_abs_err(out, exp) <= TOL["f32"]
    if D == 100:  # views of wider rows: other columns hold NaN (inputs) or a sentinel (output)
        wide = []
        for t in dev:
            w = torch.full(t.shape[:-1] + (128,), float("nan"), dtype=t.dtype, device="cuda")
            w[..., :D] = t
            wide.append(w[..., :D])
        outw = torch.full((B, Hq, L, 128), 7.0, dtype=torch.float32, device="cuda")
        rc, _ = call("forward", *wide, causal=causal, out=outw[..., :D])
        assert rc == 0 and max_abs_err(outw[..., :D], exp) <= TOL["f32"] and bool((outw[..., D:] == 7.0).all())
        m = (np.random.RandomState(D).rand(L, S) > 0.4).astype(np.uint8)
        m[:, 0] = 1
        if not causal and S % 4 == 0:
            rc, out = call("forward", *dev, mask=torch.from_numpy(m).cuda().bool())
            assert rc == 0 and max_abs_err(out, oracle.sdpa_f32(*host, mask=m)) <= TOL["f32"]


@pytest.mark.parametrize("D", [40, 80, 200])
def test_head_sizes_between_the_mfma_kernels_read_and_write_their_columns_only(D):
    # q, k, v and out are views of wider rows whose other columns hold NaN (inputs) or a sentinel (output)
    B, Hq, Hkv, L, S, W = 1, 4, 2, 150, 260, 256
    say("padded head_dim in wider rows", D)
    host, dev = make_inputs(411 + D, B, Hq, Hkv, L, S, D, "bf16", 0.7)
    wide = []
    for t in dev:
        w = torch.full(t.shape[:-1] + (W,), float("nan"), dtype=t.dtype, device="cuda")
        w[..., :D] = t
        wide.append(w[..., :D])
    exp = oracle.sdpa_f32(*host, causal=True)
    from tinytorch_amd import sdpAttention
    assert route_of(*wide, causal=True) == "prefill"
    y = sdpAttention(*wide, isCausal=True)
    assert max_abs_err(y, exp) <= TOL["bf16"]
    outw = torch.full((B, Hq, L, W), 7.0, dtype=torch.bfloat16, device="cuda")
    rc, _ = call("forward", *wide, causal=True, out=outw[..., :D])
    assert rc == 0 and max_abs_err(outw[..., :D], exp) <= TOL["bf16"] and bool((outw[..., D:] == 7.0).all())


@pytest.mark.parametrize("D,kind", [(80, "bool"), (48, "add"), (160, "bool")])
def test_head_sizes_between_the_mfma_kernels_with_masks_key_counts_and_grouped_heads(D, kind):
    B, Hq, Hkv, L, S = 2, 8, 2, 140, 264
    say("padded head_dim, mask", (D, kind))
    host, dev = make_inputs(511 + D, B, Hq, Hkv, L, S, D, "f16", 0.7)
    rng = np.random.RandomState(D)
    if kind == "bool":
        m = (rng.rand(L, S) > 0.4).astype(np.uint8)
        m[:, 1] = 1
        md = torch.from_numpy(m).cuda().bool()
    else:
        m = rng.randn(Hq, L, S).astype(np.float32)
        md = torch.from_numpy(m).cuda().half()
        m = md.float().cpu().numpy()
    assert route_of(*dev, mask=md) == "prefill"
    rc, out = call("forward", *dev, mask=md)
    assert rc == 0 and max_abs_err(out, oracle.sdpa_f32(*host, mask=m)) <= TOL["f16"]
    # per-batch key counts, bottom-right causal, few rows per head (the grouped heads of a KV head are packed into one)
    from tinytorch_amd import sdpAttention
    lens = np.array([S, 77], np.int32)
    ld = torch.from_numpy(lens).cuda()
    Lq = 5
    q = dev[0][:, :, :Lq].contiguous()
    y = sdpAttention(q, dev[1], dev[2], isCausal=True, kvLens=ld, causalAlign="bottom-right")
    for b in range(B):
        n = int(lens[b])
        mask = np.tril(np.ones((Lq, n), np.uint8), n - Lq)
        e = oracle.sdpa_f32(host[0][b:b + 1, :, :Lq], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n], mask=mask)
        assert max_abs_err(y[b:b + 1], e) <= TOL["f16"]


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_per_batch_key_counts_on_the_mfma_route(causal, dtype):
    # a padded batch: every entry has its own number of valid keys (0, 1, ragged, full)
    B, Hq, Hkv, L, S, D = 5, 4, 2, 300, 520, 128
    host, dev = make_inputs(97, B, Hq, Hkv, L, S, D, dtype)
    lens = np.array([0, 1, 77, 333, 9999], np.int32)
    ld = torch.from_numpy(lens).cuda()
    out = torch.empty_like(dev[0])
    from tinytorch_amd import _capi, build_params
    rc, r = _capi.plan(build_params(*dev, out, causal, None, None, ld))
    assert rc == 0 and _capi.ROUTE_NAMES[r] == "prefill"
    from tinytorch_amd import sdpAttention
    y = sdpAttention(*dev, isCausal=causal, kvLens=ld)
    torch.cuda.synchronize()
    assert torch.count_nonzero(y[0]) == 0
    for b in range(1, B):
        n = min(int(lens[b]), S)
        exp = oracle.sdpa_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n], causal=causal)
        assert max_abs_err(y[b:b + 1], exp) <= TOL[dtype], b


@pytest.mark.parametrize("case", [(4, 32, 8, 1, 2048, "bf16"), (2, 8, 2, 1, 33, "f16"), (3, 28, 4, 1, 777, "bf16"),
                                  (1, 16, 1, 1, 513, "bf16"), (2, 4, 1, 4, 640, "f16"), (1, 16, 2, 1, 9000, "bf16")],
                         ids=lambda c: "B%dH%dk%dL%dS%d-%s" % c)
def test_decode_head_dim_64(case):
    B, Hq, Hkv, L, S, dtype = case
    host, dev = make_inputs(99 + S, B, Hq, Hkv, L, S, 64, dtype)
    # up to 8 rows per KV head stream through the decode kernel; 9-16 take the packed-heads MFMA path when S >= 256
    assert route_of(*dev) == ("decode" if L * (Hq // Hkv) <= 8 or S < 256 else "prefill")
    exp = oracle.sdpa_f32(*host)
    rc, out = call("forward", *dev)
    assert rc == 0 and max_abs_err(out, exp) <= TOL[dtype]
    rc, out2 = call("general", *dev)
    assert rc == 0 and max_abs_err(out2, exp) <= TOL[dtype]


# ---- fp32 tensors on the fp32 matrix cores -----------------------------------------------------------------------

F32_PREFILL_CASES = [
    # B, Hq, Hkv, L, S, D, causal
    (1, 4, 4, 128, 128, 64, False),    # config 1's shape, unmasked
    (1, 8, 2, 512, 512, 128, True),    # config 3's grouping, scaled down
    (1, 7, 1, 300, 300, 128, True),    # 7 heads per KV head
    (2, 4, 2, 130, 257, 128, False),   # ragged in both directions
    (1, 2, 2, 200, 77, 64, True),      # L > S, top-left causal
    (1, 2, 2, 77, 200, 64, True),      # L < S
    (1, 3, 3, 33, 31, 128, False),     # less than one key tile
    (1, 2, 1, 1, 40, 64, False),       # a single query row
    (1, 2, 2, 5, 1, 128, True),        # a single key
    (8, 8, 8, 160, 160, 64, True),     # (batch x kv heads) multiple of 8: the XCD-aware order
]


@pytest.mark.parametrize("case", F32_PREFILL_CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-c%d" % c)
def test_fp32_mfma_prefill_against_oracle(case):
    B, Hq, Hkv, L, S, D, causal = case
    say("fp32 prefill", case)
    host, dev = make_inputs(5000 + L + S, B, Hq, Hkv, L, S, D, "f32")
    exp = oracle.sdpa_f32(*host, causal=causal)
    assert route_of(*dev, causal=causal) == "prefill"
    rc, out = call("prefill", *dev, causal=causal)
    assert rc == 0
    err = max_abs_err(out, exp)
    say("   max-abs-err", err)
    assert err <= TOL["f32"]
    rc, out2 = call("forward", *dev, causal=causal)
    assert rc == 0 and np.array_equal(to_host_f32(out2), to_host_f32(out))
    rc, out3 = call("general", *dev, causal=causal)    # the vector-ALU kernel agrees
    assert rc == 0 and max_abs_err(out3, exp) <= TOL["f32"]


def test_fp32_mfma_large_scores_views_and_scale():
    """Scores spread over hundreds of units (the running maximum has to follow every tile), a custom scale, q as a
    transposed view of a [B, L, H, D] buffer, k/v as the leading rows of a longer cache, out into a padded buffer."""
    B, Hq, Hkv, L, S, D = 2, 4, 2, 200, 333, 128
    host, dev = make_inputs(99, B, Hq, Hkv, L, S, D, "f32", mul=5.0)
    exp = oracle.sdpa_f32(*host, causal=True, scale=0.11)
    qv = dev[0].permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    kc = torch.zeros(B, Hkv, S + 50, D, device="cuda")
    vc = torch.full((B, Hkv, S + 50, D), float("nan"), device="cuda")
    kc[:, :, :S], vc[:, :, :S] = dev[1], dev[2]
    obuf = torch.full((B, Hq, L, D + 4), -7.0, device="cuda")
    ov = obuf[..., :D]
    assert route_of(qv, kc[:, :, :S], vc[:, :, :S], causal=True, scale=0.11, out=ov) == "prefill"
    rc, out = call("forward", qv, kc[:, :, :S], vc[:, :, :S], causal=True, scale=0.11, out=ov)
    assert rc == 0
    assert max_abs_err(ov, exp) <= 5.0 * TOL["f32"]     # values are 5x larger than unit-variance inputs
    assert bool((obuf[..., D:] == -7.0).all())           # nothing written outside the rows


def test_fp32_mfma_gqa_equals_repeated_kv_bitwise():
    B, Hq, Hkv, L, S, D = 1, 8, 2, 150, 150, 64
    host, dev = make_inputs(31, B, Hq, Hkv, L, S, D, "f32")
    rc, a = call("prefill", *dev, causal=True)
    G = Hq // Hkv
    rc2, b = call("prefill", dev[0], dev[1].repeat_interleave(G, 1), dev[2].repeat_interleave(G, 1), causal=True)
    assert rc == 0 and rc2 == 0
    assert torch.equal(a, b)


@pytest.mark.parametrize("mshape,kind", [((2, 1, 1, 336), "bool"), ((200, 336), "bool"), ((2, 4, 200, 336), "float"),
                                         ((4, 1, 336), "float"), ((336,), "bool"), ((200, 333), "bool"),
                                         ((2, 4, 200, 333), "float")])
@pytest.mark.parametrize("D,dtype", [(64, "f32"), (128, "f32"), (64, "bf16"), (256, "f16"), (128, "bf16")])
def test_masks_on_the_simple_mfma_kernels(mshape, kind, D, dtype):
    """attnMask on the fp32 MFMA kernel and on the 4-wavefront 16-bit kernel (head_dim != 128, or few query rows):
    every broadcastable shape, Bool and additive, against the oracle; rows whose keys are all hidden give NaN on both
    sides.  These kernels read the mask four keys at a time; a key count that is not a multiple of 4 goes to the
    vector-ALU kernel (the pipelined head_dim-128 kernel takes any mask)."""
    S = mshape[-1]
    B, Hq, Hkv, L = 2, 4, 2, (200 if not (D == 128 and dtype == "bf16") else 100)
    if len(mshape) >= 2 and mshape[-2] == 200:
        mshape = mshape[:-2] + (L, S)
    say("mask on simple mfma kernels", mshape, kind, D, dtype)
    host, dev = make_inputs(6100 + D, B, Hq, Hkv, L, S, D, dtype)
    rng = np.random.default_rng(len(mshape) * 10 + D)
    if kind == "bool":
        m = (rng.random(mshape) > 0.3)
        m[..., 0] = True                     # at least one visible key per row
        if len(mshape) >= 2 and mshape[-2] == L:
            m[..., 5, :] = False              # except one row, hidden entirely
        mh, md = m.astype(np.uint8), torch.from_numpy(m).cuda()
    else:
        mv, mb = oracle.round_to(rng.standard_normal(mshape).astype(np.float32) * 2, dtype)
        mh, md = mv, to_device(mv, mb, dtype)
    exp = oracle.sdpa_f32(*host, mask=mh)
    assert route_of(*dev, mask=md) == ("prefill" if S % 4 == 0 else "general")
    rc, out = call("forward", *dev, mask=md)
    assert rc == 0
    y = to_host_f32(out)
    assert np.array_equal(np.isnan(y), np.isnan(exp))
    ok = ~np.isnan(exp)
    assert np.abs(y[ok] - exp[ok]).max() <= TOL[dtype]


@pytest.mark.parametrize("causal", [False, True])
def test_fp32_mfma_per_batch_key_counts(causal):
    B, Hq, Hkv, L, S, D = 4, 4, 2, 150, 400, 128
    host, dev = make_inputs(6200, B, Hq, Hkv, L, S, D, "f32")
    lens = [400, 137, 0, 9999]
    kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
    assert route_of(*dev, causal=causal, kv_lens=kv) == "prefill"
    rc, out = call("forward", *dev, causal=causal, kv_lens=kv)
    assert rc == 0
    for b, n in enumerate(lens):
        n = min(n, S)
        if n == 0:
            assert torch.count_nonzero(out[b]) == 0
            continue
        exp = oracle.sdpa_f32(host[0][b:b + 1], host[1][b:b + 1, :, :n], host[2][b:b + 1, :, :n], causal=causal)
        assert max_abs_err(out[b:b + 1], exp) <= TOL["f32"], b
