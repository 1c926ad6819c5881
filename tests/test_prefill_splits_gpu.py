"""Key splits of the pipelined prefill kernels (head_dim 128 and 64): calls with at most a quarter as many 256-row tiles as the chip
has CUs (a chunk of rows against a long cache, a few heads) divide the keys of a row tile among workgroups, and the decode path's merge kernel combines their
records.  ttsdpa_forward with its workspace takes that form; ttsdpa_prefill (no workspace) runs the same call unsplit:
both against the oracle, and against each other.  The records are combined by the kernel file's own merge kernel."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import TOL, call, make_inputs, route_of
from test_prefill_d64_gpu import sampled_rows_err
from tinytorch_amd import _capi
from tinytorch_amd.function import build_params

pytestmark = pytest.mark.gpu


def workspace_bytes(q, k, v, **kw):
    out = torch.empty_like(q)
    p = build_params(q, k, v, out, kw.get("causal", False), None, None, kw.get("kv_lens"), kw.get("align", "top-left"), None)
    return _capi.lib().ttsdpa_workspace_bytes(ctypes.byref(p))


CASES = [
    # B, Hq, Hkv, L, S, causal, align, dtype
    (1, 2, 2, 8192, 8192, True, "top-left", "bf16"),      # two heads of one long sequence
    (2, 4, 1, 4096, 4096, True, "top-left", "bf16"),      # one KV head's share of config 3 (128 row tiles, causal)
    (2, 4, 1, 2048, 8192, True, "bottom-right", "bf16"),  # a 2048-row chunk of one KV head's share of a model
    (1, 8, 8, 1024, 16384, False, "top-left", "bf16"),
    (1, 8, 2, 700, 5000, True, "bottom-right", "f16"),    # a ragged chunk at the end of a ragged cache
    (1, 6, 2, 1500, 3333, False, "top-left", "f16"),
    (1, 2, 1, 300, 20000, True, "bottom-right", "bf16"),  # many splits of a short chunk
]


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%dH%dk%dL%dS%d-c%d-%s-%s" % c)
def test_split_keys_against_oracle_and_unsplit(case, D):
    B, Hq, Hkv, L, S, causal, align, dtype = case
    host, dev = make_inputs(9000 + L + S + D, B, Hq, Hkv, L, S, D, dtype, 0.8)
    assert route_of(*dev, causal=causal, align=align) == "prefill"
    assert workspace_bytes(*dev, causal=causal, align=align) >= 2 * B * Hq * L * (D + 2) * 4   # at least two records per row
    rc, split = call("forward", *dev, causal=causal, align=align)
    assert rc == 0
    rc, whole = call("prefill", *dev, causal=causal, align=align)
    assert rc == 0
    d = (split.float() - whole.float()).abs().max().item()
    assert d <= 1e-2, d   # the same arithmetic in another order, rounded to 16 bits once
    rows = [(0, 0), (B - 1, Hq - 1)]
    assert sampled_rows_err(split, host, causal, rows, align=align) <= TOL[dtype]


def test_split_keys_with_per_batch_key_counts():
    B, Hq, Hkv, L, S = 3, 4, 2, 1024, 6000
    host, dev = make_inputs(9911, B, Hq, Hkv, L, S, 128, "bf16", 0.8)
    lens = np.array([6000, 0, 1300], np.int32)
    kv = torch.from_numpy(lens).cuda()
    for causal in (False, True):
        out = torch.full(dev[0].shape, 7.0, dtype=dev[0].dtype, device="cuda")
        rc, out = call("forward", *dev, causal=causal, align="bottom-right", kv_lens=kv, out=out)
        assert rc == 0
        assert torch.count_nonzero(out[1]).item() == 0   # no keys: zeros, from the merge kernel
        rc, whole = call("prefill", *dev, causal=causal, align="bottom-right", kv_lens=kv)
        assert rc == 0
        assert (out.float() - whole.float()).abs().max().item() <= 1e-2
        assert sampled_rows_err(out, host, causal, [(0, 1), (2, 3)], align="bottom-right", kv_len=lens) <= TOL["bf16"]
