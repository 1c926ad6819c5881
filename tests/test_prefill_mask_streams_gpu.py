"""Bool attnMasks applied inside the pipelined kernels' instruction streams (head_dim 128 and 64: a wavefront's mask bytes
of a tile brought into LDS two tiles ahead, a byte compare and a select per probability): against the oracle, which
restates the reference's masked fill and broadcasting add (reference src/Function/FuncNNLayer.h:249-260)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import TOL, call, make_inputs, max_abs_err, route_of, to_host_f32

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def bool_mask(seed, shape, keep=0.6):
    m = (np.random.RandomState(seed).rand(*shape) < keep).astype(np.uint8)
    m[..., 1] = 1  # no row without a visible key
    return m


@pytest.mark.parametrize("case", [
    # B, Hq, Hkv, L, S, mask shape, dtype
    (1, 2, 2, 512, 2048, (512, 2048), "bf16"),            # many tiles in the pipelined form
    (2, 4, 2, 300, 1024, (2, 4, 300, 1024), "f16"),       # a mask per (batch, head), ragged last row tile
    (2, 4, 1, 257, 1000, (2, 1, 1, 1000), "bf16"),        # key padding; keys not a multiple of the 64-key tile
    (1, 4, 4, 600, 164, (4, 600, 164), "bf16"),           # the shortest rows that still have a tile in that form
    (1, 2, 2, 384, 156, (384, 156), "f16"),               # below it: every step in the general form
    (1, 3, 1, 1024, 4096, (1024, 4096), "bf16"),          # grouped heads, long rows
    # (the head_dim-64 pipelined kernel takes calls of 512 rows and more)
    (2, 4, 2, 700, 1024, (2, 4, 700, 1024), "f16"),       # a mask per (batch, head), ragged last row tile
    (2, 4, 1, 513, 1000, (2, 1, 1, 1000), "bf16"),        # key padding; keys not a multiple of the 64-key tile
    (1, 2, 2, 640, 156, (640, 156), "f16"),               # every step in the general form
], ids=lambda c: "B%dH%dk%dL%dS%d-m%s-%s" % (c[0], c[1], c[2], c[3], c[4], "x".join(map(str, c[5])), c[6]))
@pytest.mark.parametrize("D", [128, 64])
def test_bool_mask_in_streams_against_oracle(case, D):
    B, Hq, Hkv, L, S, mshape, dtype = case
    say("bool mask in streams", case, D)
    host, dev = make_inputs(700 + L + S + D, B, Hq, Hkv, L, S, D, dtype)
    m = bool_mask(L + S, mshape)
    md = torch.from_numpy(m).cuda().bool()
    assert route_of(*dev, mask=md) == "prefill"
    exp = oracle.sdpa_f32(*host, mask=m)
    rc, out = call("forward", *dev, mask=md)
    assert rc == 0
    err = max_abs_err(out, exp)
    say("   max-abs-err", err)
    assert err <= TOL[dtype]


@pytest.mark.parametrize("D", [128, 64])
def test_hidden_scores_do_not_enter_the_maximum(D):
    """Large scores behind cleared mask bytes: the maximum the exponentials are taken against is raised from visible
    scores only (a hidden score of 300 would flush every visible probability to zero), also where it is raised inside
    the pipelined form."""
    B, Hq, Hkv, L, S = 1, 2, 2, 512, 1024
    say("hidden large scores", D)
    host, dev = make_inputs(733, B, Hq, Hkv, L, S, D, "bf16", 0.5 if D == 128 else 0.7)
    q, k, v = host
    k = k.copy()
    rng = np.random.RandomState(5)
    hot = rng.choice(S, 40, replace=False)
    k[:, :, hot] *= 24.0        # scores of these keys are ~24 times larger: far above the others
    kv, kb = oracle.round_to(k, "bf16")
    m = bool_mask(9, (L, S), 0.7)
    m[:, hot[:30]] = 0          # most of the hot keys are hidden ...
    m[::3, hot[30:]] = 0        # ... the rest only for every third row: the other rows do have to raise their maximum
    from gpu_util import to_device
    dev = (dev[0], to_device(kv, kb, "bf16"), dev[2])
    md = torch.from_numpy(m).cuda().bool()
    exp = oracle.sdpa_f32(q, kv, v, mask=m)
    rc, out = call("forward", *dev, mask=md)
    assert rc == 0 and np.isfinite(exp).all()
    err = max_abs_err(out, exp)
    say("   hidden large scores: max-abs-err", err)
    assert err <= TOL["bf16"]
    rc, out2 = call("general", *dev, mask=md)
    assert rc == 0 and np.abs(to_host_f32(out) - to_host_f32(out2)).max() <= 2e-2


@pytest.mark.parametrize("D", [128, 64])
def test_fully_hidden_rows_and_views(D):
    B, Hq, Hkv, L, S = 2, 4, 2, 520, 640
    say("fully hidden rows, mask views", D)
    host, dev = make_inputs(741, B, Hq, Hkv, L, S, D, "bf16")
    m = bool_mask(3, (B, 1, L, S))
    m[0, 0, 17] = 0             # rows without a visible key: NaN in the reference (0 * inf)
    m[1, 0, 300:333] = 0
    m[1, 0, 511, 64:] = 0       # a row that only sees its first tile
    md = torch.from_numpy(m).cuda().bool()
    exp = oracle.sdpa_f32(*host, mask=m)
    rc, out = call("forward", *dev, mask=md)
    y = to_host_f32(out)
    assert rc == 0 and np.array_equal(np.isnan(y), np.isnan(exp)) and np.isnan(exp[0, :, 17]).all()
    ok = ~np.isnan(exp)
    assert np.abs(y[ok] - exp[ok]).max() <= TOL["bf16"]
    # an expanded view (head stride 0) and a sliced view of a larger mask (row pitch beyond the row) give the same
    rc, out_e = call("forward", *dev, mask=md.expand(B, Hq, L, S))
    assert rc == 0 and torch.equal(torch.nan_to_num(out_e.float()), torch.nan_to_num(out.float()))
    big = torch.zeros(B, 1, L, 2 * S, dtype=torch.bool, device="cuda")
    big[..., :S] = md
    rc, out_s = call("forward", *dev, mask=big[..., :S])
    assert rc == 0 and torch.equal(torch.nan_to_num(out_s.float()), torch.nan_to_num(out.float()))
    # a view whose rows start at a byte that is not a multiple of 4 leaves the streams (element loads): same values
    rc, out_o = call("forward", *dev, mask=torch.cat([big[..., :1], big], dim=-1)[..., 1:S + 1])
    assert rc == 0 and np.abs(np.nan_to_num(to_host_f32(out_o)) - np.nan_to_num(y)).max() <= 1e-2
