"""The pipelined prefill kernel at head_dim 64 (csrc/sdpa_prefill_d64.hip) against the oracle: it takes calls without an
attnMask or pages of 512 query rows and more, or shorter ones that fill half of the chip's CUs with 256-row workgroups, so
its cases are larger than the other parity tests'.  Smaller head_dim-64 calls keep running on the 4-wavefront kernel and
are covered in test_parity_gpu.py; both kernels must agree with the oracle on the same inputs."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, call, make_inputs, max_abs_err, route_of, to_host_f32

pytestmark = pytest.mark.gpu


def sampled_rows_err(out_dev, host, causal, rows, align="top-left", kv_len=None):
    """max-abs-error of the sampled (batch, head) slices against the oracle"""
    q, k, v = host
    B, Hq, L, D = q.shape
    G = Hq // k.shape[1]
    y = to_host_f32(out_dev)
    worst = 0.0
    for b, h in rows:
        S = k.shape[2] if kv_len is None else int(kv_len[b])
        kk, vv = k[b:b + 1, h // G:h // G + 1, :S], v[b:b + 1, h // G:h // G + 1, :S]
        if align == "bottom-right" and causal:
            i = np.arange(L)[:, None]
            j = np.arange(S)[None, :]
            mask = j <= i + max(0, S - L)
            exp = oracle.sdpa_f32(q[b:b + 1, h:h + 1], kk, vv, causal=False, mask=mask)
        else:
            exp = oracle.sdpa_f32(q[b:b + 1, h:h + 1], kk, vv, causal=causal)
        got = y[b:b + 1, h:h + 1]
        assert np.isfinite(got).all()
        worst = max(worst, float(np.abs(got.astype(np.float64) - exp.astype(np.float64)).max()))
    return worst


ROWS = [(0, 0), (0, 5), (1, 17), (1, 63), (3, 31)]


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal,L,S", [(True, 500, 500), (True, 769, 769), (False, 320, 411), (False, 257, 64)])
def test_head_dim_64_pipelined_against_oracle(dtype, D, causal, L, S):
    # (head_dim 128 rides along: its pipelined kernel with this many workgroups takes the causal row tiles in mirror
    # pairs, which the smaller shapes of the other parity tests do not)
    B, Hq, Hkv = 4, 64, 16
    host, dev = make_inputs(640 + L + D, B, Hq, Hkv, L, S, D, dtype, 0.8)
    assert route_of(*dev, causal=causal) == "prefill"
    rc, out = call("forward", *dev, causal=causal)
    assert rc == 0
    assert sampled_rows_err(out, host, causal, ROWS) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_head_dim_64_pipelined_bottom_right_and_key_counts(dtype):
    B, Hq, Hkv, L, S, D = 4, 64, 64, 300, 700, 64
    host, dev = make_inputs(777, B, Hq, Hkv, L, S, D, dtype, 0.8)
    rc, out = call("forward", *dev, causal=True, align="bottom-right")
    assert rc == 0
    assert sampled_rows_err(out, host, True, ROWS, align="bottom-right") <= TOL[dtype]
    lens = np.array([700, 333, 64, 1], np.int32)
    rc, out = call("forward", *dev, causal=False, kv_lens=torch.from_numpy(lens).cuda())
    assert rc == 0
    assert sampled_rows_err(out, host, False, ROWS, kv_len=lens) <= TOL[dtype]
    rc, out = call("forward", *dev, causal=True, align="bottom-right", kv_lens=torch.from_numpy(lens).cuda())
    assert rc == 0
    assert sampled_rows_err(out, host, True, ROWS, align="bottom-right", kv_len=lens) <= TOL[dtype]


def test_head_dim_64_pipelined_equals_the_4_wavefront_kernel_within_rounding():
    # the same call through both kernels: causal on the pipelined kernel, and the same triangle as an additive attnMask
    # (0 / -inf), which the pipelined kernel does not take (one batch entry: the other kernel reads the mask from memory)
    B, Hq, Hkv, L, S, D = 4, 64, 16, 512, 512, 64
    host, dev = make_inputs(4242, B, Hq, Hkv, L, S, D, "bf16", 0.8)
    rc, big = call("forward", *dev, causal=True)
    assert rc == 0
    tril = torch.ones(L, S, dtype=torch.bool, device="cuda").tril()
    first = (dev[0][:1].contiguous(), dev[1][:1].contiguous(), dev[2][:1].contiguous())
    bias = torch.zeros(L, S, dtype=torch.bfloat16, device="cuda").masked_fill(~tril, float("-inf"))
    rc, one = call("forward", *first, mask=bias)
    assert rc == 0
    d = (big[:1].float() - one.float()).abs().max().item()
    assert 0 < d <= 2e-2   # two kernels: close, not identical
    # the triangle as a Bool attnMask runs in the pipelined kernel's streams like the causal flag
    rc, two = call("forward", *first, mask=tril)
    assert rc == 0 and (big[:1].float() - two.float()).abs().max().item() <= 2e-2
    # causal row 0 is v[0] exactly on both
    assert torch.equal(big[:, :, 0, :], dev[2][:, :, 0, :].repeat_interleave(Hq // Hkv, dim=1))
    assert torch.equal(one[:, :, 0, :], dev[2][:1, :, 0, :].repeat_interleave(Hq // Hkv, dim=1))


def test_large_score_range_head_dim_64_pipelined():
    # scores far apart: the lazily raised maximum must not lose the small probabilities nor overflow the large ones
    B, Hq, Hkv, L, S, D = 4, 64, 16, 300, 300, 64
    host, dev = make_inputs(99, B, Hq, Hkv, L, S, D, "bf16", 6.0)
    rc, out = call("forward", *dev, causal=True)
    assert rc == 0
    assert sampled_rows_err(out, host, True, ROWS) <= 0.12


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("S", [1, 31, 33, 65, 130, 191])
def test_head_dim_64_pipelined_few_keys(causal, S):
    # fewer keys than the ring of tiles holds, down to one: ragged first tile, no steady state at all
    B, Hq, Hkv, L, D = 8, 32, 8, 200, 64
    host, dev = make_inputs(900 + S, B, Hq, Hkv, L, S, D, "bf16", 0.8)
    assert route_of(*dev, causal=causal) == "prefill"
    rc, out = call("forward", *dev, causal=causal)
    assert rc == 0
    rows = [(0, 0), (3, 9), (7, 31)]
    assert sampled_rows_err(out, host, causal, rows) <= TOL["bf16"]


def test_head_dim_64_pipelined_empty_cache_entries_give_zeros():
    B, Hq, Hkv, L, S, D = 8, 32, 8, 200, 96, 64
    host, dev = make_inputs(31337, B, Hq, Hkv, L, S, D, "bf16", 0.8)
    lens = np.array([96, 0, 5, 0, 64, 65, 0, 96], np.int32)
    out = torch.full(dev[0].shape, 7.0, dtype=dev[0].dtype, device="cuda")
    rc, out = call("forward", *dev, causal=False, kv_lens=torch.from_numpy(lens).cuda(), out=out)
    assert rc == 0
    for b in (1, 3, 6):
        assert torch.count_nonzero(out[b]).item() == 0
    assert sampled_rows_err(out, host, False, [(0, 0), (2, 7), (4, 30), (5, 1), (7, 31)], kv_len=lens) <= TOL["bf16"]


def test_head_dim_64_pipelined_strided_views_equal_contiguous_bitwise():
    # q, k, v as views of one packed [B, L, 3, H, D] projection output: only the row stride differs
    B, H, L, D = 4, 64, 300, 64
    host, dev = make_inputs(2024, B, H, H, L, L, D, "f16", 0.8)
    packed = torch.empty(B, L, 3, H, D, dtype=dev[0].dtype, device="cuda")
    for i in range(3):
        packed[:, :, i] = dev[i].permute(0, 2, 1, 3)
    views = [packed[:, :, i].permute(0, 2, 1, 3) for i in range(3)]
    assert not views[0].is_contiguous()
    assert route_of(*views, causal=True) == "prefill"
    rc, a = call("forward", *dev, causal=True)
    assert rc == 0
    rc, b = call("forward", *views, causal=True)
    assert rc == 0
    assert torch.equal(a, b)
    # and into a strided output
    outp = torch.zeros(B, L, H, D, dtype=dev[0].dtype, device="cuda")
    rc, c = call("forward", *views, causal=True, out=outp.permute(0, 2, 1, 3))
    assert rc == 0
    assert torch.equal(a, outp.permute(0, 2, 1, 3))


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("B,L,S,align", [(1, 900, 900, "top-left"), (2, 600, 1000, "bottom-right"), (1, 4200, 4200, "top-left")])
def test_pipelined_single_row_tiles(D, B, L, S, align):
    # fewer mirror pairs than CUs (or a last round far from full): one causal row tile per workgroup, longest first
    Hq, Hkv = 64, 16
    if L > 4000:
        Hq, Hkv = 40, 8   # 40 heads x 17 tiles: 360 pairs, 1.4 rounds of the chip
    host, dev = make_inputs(8100 + L + D, B, Hq, Hkv, L, S, D, "bf16", 0.8)
    assert route_of(*dev, causal=True, align=align) == "prefill"
    rc, out = call("forward", *dev, causal=True, align=align)
    assert rc == 0
    rows = [(0, 0), (0, 5), (B - 1, 17), (B - 1, Hq - 1)] if L < 4000 else [(0, 3), (0, Hq - 1)]
    assert sampled_rows_err(out, host, True, rows, align=align) <= TOL["bf16"]
