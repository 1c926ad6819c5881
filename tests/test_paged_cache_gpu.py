"""Paged KV cache (block tables over page pools): the same attention as over contiguous K/V, which is what the oracle
computes.  The reference has neither a cache nor pages; a caller's K/V there are contiguous tensors grown with
op::concat (reference src/Operation/OpTransform.cpp:306-357)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, TORCH_DTYPE, call, make_inputs, max_abs_err, route_of, to_host_f32
from tinytorch_amd import kvCacheAppend, sdpAttention

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def scatter_to_pages(kd, vd, page, seed, spare=3):
    """Contiguous [B,Hkv,S,D] -> (k pool, v pool [P,Hkv,page,D], block table int32 [B, n]) with the pages of all batch
    entries shuffled through the pool; unused pool pages hold NaN."""
    B, Hkv, S, D = kd.shape
    n = (S + page - 1) // page
    P = B * n + spare
    perm = torch.from_numpy(np.random.default_rng(seed).permutation(P)[:B * n].astype(np.int32)).cuda()
    table = perm.view(B, n).contiguous()
    kp = torch.full((P, Hkv, page, D), float("nan"), dtype=kd.dtype, device="cuda")
    vp = torch.full_like(kp, float("nan"))
    for b in range(B):
        for j in range(n):
            rows = min(page, S - j * page)
            pg = int(table[b, j])
            kp[pg, :, :rows] = kd[b, :, j * page:j * page + rows]
            vp[pg, :, :rows] = vd[b, :, j * page:j * page + rows]
            kp[pg, :, rows:] = 0   # the tail of a last page is never attended to, but must not poison 0 * x
            vp[pg, :, rows:] = 0
    return kp, vp, table


CASES = [
    # B, Hq, Hkv, L, S, D, dtype, page, route
    (4, 8, 2, 1, 2048, 128, "bf16", 64, "decode"),
    (2, 32, 8, 1, 8192, 128, "bf16", 256, "decode"),     # split cache + merge
    (3, 8, 4, 1, 1000, 64, "f16", 32, "decode"),         # ragged last page, head_dim 64
    (2, 8, 2, 2, 3000, 128, "bf16", 128, "decode"),      # 8 rows per KV head
    (2, 8, 2, 4, 3000, 128, "bf16", 128, "prefill"),     # 16 rows per KV head: packed heads on the MFMA kernel
    (2, 8, 2, 4, 3000, 128, "bf16", 32, "decode"),       # ... or the streaming kernel when the pages are too small for it
    (2, 4, 2, 1, 300, 128, "bf16", 16, "general"),       # pages smaller than a key block
    (2, 4, 2, 40, 200, 96, "f32", 8, "general"),
    (1, 4, 4, 70, 500, 128, "f16", 64, "prefill"),       # many query rows: the 4-wavefront MFMA kernel, ragged last tile
    (1, 4, 4, 70, 500, 128, "f16", 32, "general"),       # ... whose 64-key tiles need pages of 64 rows or more
    (2, 8, 2, 300, 1500, 128, "bf16", 128, "prefill"),   # the pipelined head_dim-128 kernel over pages
    (2, 8, 4, 200, 777, 64, "bf16", 64, "prefill"),      # head_dim 64, ragged last page
    (2, 4, 2, 130, 600, 96, "f16", 256, "prefill"),      # head_dim 96
    (2, 8, 2, 150, 900, 128, "f32", 64, "prefill"),      # the fp32 MFMA kernel
    (2, 8, 4, 1, 2000, 64, "f32", 128, "prefill"),       # fp32 decode: packed heads + split keys over pages
    (2, 32, 8, 8, 4096, 128, "bf16", 256, "prefill"),    # 32 rows per KV head: packed heads + split keys over pages
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-%s-p%d-%s" % c)
def test_paged_attention_against_oracle(case):
    B, Hq, Hkv, L, S, D, dtype, page, route = case
    say("paged", case)
    host, dev = make_inputs(9000 + S + page, B, Hq, Hkv, L, S, D, dtype)
    kp, vp, table = scatter_to_pages(dev[1], dev[2], page, seed=S)
    lens = torch.full((B,), S, dtype=torch.int32, device="cuda")
    exp = oracle.sdpa_f32(*host)
    out = sdpAttention(dev[0], kp, vp, kvLens=lens, blockTable=table)
    assert max_abs_err(out, exp) <= TOL[dtype]
    o2 = torch.empty_like(dev[0])
    assert route_of(dev[0], kp, vp, kv_lens=lens, block_table=table, out=o2) == route
    rc, o3 = call("general", dev[0], kp, vp, kv_lens=lens, block_table=table)   # the vector-ALU kernel agrees
    assert rc == 0 and max_abs_err(o3, exp) <= TOL[dtype]


@pytest.mark.parametrize("dtype,D,page", [("bf16", 128, 64), ("f16", 64, 32), ("f32", 96, 16)])
def test_paged_generation_loop(dtype, D, page):
    """Append into pages and attend over per-batch lengths, several steps, one and several new tokens per step
    (bottom-right causal for the latter) — against the oracle on the contiguous history."""
    B, Hq, Hkv, Smax = 3, 8, 2, 512
    say("paged generation", dtype, D, page)
    td = TORCH_DTYPE[dtype]
    host, dev = make_inputs(9500 + D, B, Hq, Hkv, 8, Smax, D, dtype)   # q rows are drawn from host[0] per step
    kall, vall = dev[1], dev[2]
    n = Smax // page
    P = B * n + 2
    perm = torch.from_numpy(np.random.default_rng(D).permutation(P)[:B * n].astype(np.int32)).cuda().view(B, n).contiguous()
    kp = torch.zeros(P, Hkv, page, D, dtype=td, device="cuda")
    vp = torch.zeros_like(kp)
    lens = [200, 37, 0]
    for b in range(B):   # prompts of different lengths, appended per batch entry
        if lens[b]:
            kvCacheAppend(kp, vp, kall[b:b + 1, :, :lens[b]], vall[b:b + 1, :, :lens[b]], 0, blockTable=perm[b:b + 1])
    for step, new in enumerate((1, 3, 1, 2)):
        pos = torch.tensor(lens, dtype=torch.int32, device="cuda")
        kn = torch.stack([kall[b, :, lens[b]:lens[b] + new] for b in range(B)])
        vn = torch.stack([vall[b, :, lens[b]:lens[b] + new] for b in range(B)])
        kvCacheAppend(kp, vp, kn, vn, pos, blockTable=perm)
        lens = [x + new for x in lens]
        kv = torch.tensor(lens, dtype=torch.int32, device="cuda")
        q = dev[0][:, :, :new]
        out = sdpAttention(q, kp, vp, isCausal=new > 1, causalAlign="bottom-right", kvLens=kv, blockTable=perm)
        for b in range(B):
            m = (np.arange(lens[b])[None, :] <= np.arange(new)[:, None] + lens[b] - new).astype(np.uint8)
            exp = oracle.sdpa_f32(host[0][b:b + 1, :, :new], host[1][b:b + 1, :, :lens[b]], host[2][b:b + 1, :, :lens[b]], mask=m)
            assert max_abs_err(out[b:b + 1], exp) <= TOL[dtype], (step, b)
    # every page holds exactly the rows of the contiguous history it maps to
    for b in range(B):
        for j in range((lens[b] + page - 1) // page):
            rows = min(page, lens[b] - j * page)
            assert torch.equal(kp[int(perm[b, j]), :, :rows], kall[b, :, j * page:j * page + rows])
            assert torch.equal(vp[int(perm[b, j]), :, :rows], vall[b, :, j * page:j * page + rows])


def test_paged_equals_contiguous_bitwise_at_full_size():
    """Config 4's shape: the decode kernel over pages of 256 rows gives the bits it gives over the contiguous cache
    (same blocks, same order; only the addresses differ)."""
    B, Hq, Hkv, S, D, page = 64, 32, 8, 8192, 128, 256
    gen = torch.Generator(device="cuda").manual_seed(5)
    q = torch.randn(B, Hq, 1, D, device="cuda", generator=gen).bfloat16()
    k = torch.randn(B, Hkv, S, D, device="cuda", generator=gen).bfloat16()
    v = torch.randn(B, Hkv, S, D, device="cuda", generator=gen).bfloat16()
    n = S // page
    perm = torch.randperm(B * n, device="cuda", generator=gen).int().view(B, n).contiguous()
    kp = torch.empty(B * n, Hkv, page, D, dtype=torch.bfloat16, device="cuda")
    vp = torch.empty_like(kp)
    kp[perm.view(-1).long()] = k.view(B, Hkv, n, page, D).permute(0, 2, 1, 3, 4).reshape(B * n, Hkv, page, D)
    vp[perm.view(-1).long()] = v.view(B, Hkv, n, page, D).permute(0, 2, 1, 3, 4).reshape(B * n, Hkv, page, D)
    ref = sdpAttention(q, k, v)
    out = sdpAttention(q, kp, vp, blockTable=perm)
    assert torch.equal(ref, out)


def test_paged_chunked_prefill_equals_contiguous_bitwise():
    """Config 3's shape as four chunks of 1024 tokens: each chunk's K/V rows are appended into pages of 128 rows, then
    its queries attend bottom-right causally to the cache so far.  The pipelined kernel over pages gives the bits it
    gives over the contiguous prefix (same tiles, same order; only the tile addresses differ)."""
    B, Hq, Hkv, S, D, C, page = 2, 32, 8, 4096, 128, 1024, 128
    gen = torch.Generator(device="cuda").manual_seed(12)
    q = torch.randn(B, Hq, S, D, device="cuda", generator=gen).bfloat16()
    k = torch.randn(B, Hkv, S, D, device="cuda", generator=gen).bfloat16()
    v = torch.randn(B, Hkv, S, D, device="cuda", generator=gen).bfloat16()
    n = S // page
    table = torch.randperm(B * n + 5, device="cuda", generator=gen)[:B * n].int().view(B, n).contiguous()
    kp = torch.full((B * n + 5, Hkv, page, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    vp = torch.full_like(kp, float("nan"))
    for c in range(S // C):
        say("paged chunk", c)
        end = (c + 1) * C
        kvCacheAppend(kp, vp, k[:, :, c * C:end], v[:, :, c * C:end], c * C, blockTable=table)
        lens = torch.full((B,), end, dtype=torch.int32, device="cuda")
        qc = q[:, :, c * C:end]
        o = torch.empty_like(qc)
        assert route_of(qc, kp, vp, kv_lens=lens, block_table=table, out=o, causal=True, align="bottom-right") == "prefill"
        paged = sdpAttention(qc, kp, vp, isCausal=True, causalAlign="bottom-right", kvLens=lens, blockTable=table)
        flat = sdpAttention(qc, k[:, :, :end], v[:, :, :end], isCausal=True, causalAlign="bottom-right")
        assert torch.equal(paged, flat), c
