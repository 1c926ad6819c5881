"""Pins the oracle's attention gradients.  The reference implements no backward for attention or matmul (reference
src/Function/FuncNNLayer.h:267, src/Function/FuncLinalg.h:20), so there is no vector of its own to compare with:
the gradients are held to central differences of an independent float64 forward (itself held to the pinned forward
oracle), to closed forms and to invariants, chosen so that a dropped term, a wrong sign or a transposed operand fails."""
import numpy as np
import pytest

import oracle


def forward64(q, k, v, causal=False, scale=None, mask=None):
    """Plain float64 attention, written independently of the oracle's loops."""
    B, Hq, L, D = q.shape
    Hkv, S = k.shape[1], k.shape[2]
    G = Hq // Hkv
    sc = 1.0 / np.sqrt(D) if scale is None else float(scale)
    kk = np.repeat(k.astype(np.float64), G, axis=1)
    vv = np.repeat(v.astype(np.float64), G, axis=1)
    s = np.einsum("bhld,bhsd->bhls", q.astype(np.float64), kk) * sc
    if causal:
        s = np.where(np.arange(S)[None, :] <= np.arange(L)[:, None], s, -np.inf)
    if mask is not None:
        s = np.where(mask, s, -np.inf) if mask.dtype == np.bool_ else s + mask
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bhls,bhsd->bhld", p, vv)


def numeric_grad(f, x, dout, h=1e-5):
    """d/dx of sum(f(x) * dout) by central differences, every element."""
    g = np.zeros_like(x, dtype=np.float64)
    flat = x.reshape(-1)
    for i in range(flat.size):
        old = flat[i]
        flat[i] = old + h
        up = (f() * dout).sum()
        flat[i] = old - h
        dn = (f() * dout).sum()
        flat[i] = old
        g.reshape(-1)[i] = (up - dn) / (2 * h)
    return g


def inputs(seed, B, Hq, Hkv, L, S, D):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((B, Hq, L, D)), rng.standard_normal((B, Hkv, S, D)), rng.standard_normal((B, Hkv, S, D)),
            rng.standard_normal((B, Hq, L, D)))


CASES = [
    # B, Hq, Hkv, L, S, D, causal, mask
    (1, 1, 1, 3, 4, 2, False, None),
    (2, 2, 2, 4, 4, 3, True, None),
    (1, 4, 2, 3, 5, 4, False, None),       # grouped heads: dk / dv sum over the group
    (1, 2, 1, 5, 3, 2, True, None),        # L > S, causal top-left
    (1, 2, 2, 3, 4, 3, False, "bool"),
    (2, 2, 1, 3, 4, 2, False, "float"),
    (2, 4, 2, 2, 3, 2, False, "bool4d"),   # mask broadcast over [B,1,L,S]
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%dH%dk%dL%dS%dD%d-c%d-%s" % c)
def test_gradients_match_central_differences(case):
    B, Hq, Hkv, L, S, D, causal, mk = case
    q, k, v, dout = inputs(sum(case[:6]), B, Hq, Hkv, L, S, D)
    q, k, v, dout = [x.astype(np.float32).astype(np.float64) for x in (q, k, v, dout)]
    rng = np.random.default_rng(7)
    mask = None
    if mk == "bool":
        mask = rng.random((L, S)) < 0.6
        mask[:, 0] = True   # no fully hidden row
    elif mk == "float":
        mask = rng.standard_normal((L, S)).astype(np.float32)
    elif mk == "bool4d":
        mask = rng.random((B, 1, L, S)) < 0.6
        mask[..., 0] = True
    scale = 0.7
    # the float64 forward is the function the pinned forward oracle computes
    got = oracle.sdpa_f32(q, k, v, causal=causal, scale=scale, mask=mask)
    assert np.abs(got - forward64(q, k, v, causal, scale, mask)).max() < 2e-6
    dq, dk, dv = oracle.sdpa_backward_f32(q, k, v, dout, causal=causal, scale=scale, mask=mask)
    f = lambda: forward64(q, k, v, causal, scale, mask)
    for name, x, g in (("dq", q, dq), ("dk", k, dk), ("dv", v, dv)):
        num = numeric_grad(f, x, dout)
        assert np.abs(num - g).max() < 1e-5 * max(1.0, np.abs(num).max()), name


def test_one_key_closed_form():
    """S == 1: P == 1 whatever the scores, so out = v[0]: dq = 0, dk = 0, dv = sum over rows (and group heads) of dout."""
    q, k, v, dout = inputs(3, 2, 4, 2, 5, 1, 8)
    dq, dk, dv = oracle.sdpa_backward_f32(q, k, v, dout)
    assert np.all(dq == 0) and np.all(dk == 0)
    exp = dout.reshape(2, 2, 2, 5, 8).sum(axis=(2, 3))[:, :, None, :]
    assert np.abs(dv - exp).max() < 1e-5


def test_zero_queries_closed_form():
    """q == 0: P is uniform (1/S).  dv_j = mean weight * sum_i dout_i; dk = 0 (it is scale * dS^T q);
    dq_i = scale * sum_j (1/S) (dP_ij - mean_j dP_ij) k_j with dP = dout v^T."""
    B, H, L, S, D = 1, 2, 3, 6, 4
    _, k, v, dout = inputs(4, B, H, H, L, S, D)
    k, v, dout = [x.astype(np.float32).astype(np.float64) for x in (k, v, dout)]
    q = np.zeros((B, H, L, D))
    sc = 0.3
    dq, dk, dv = oracle.sdpa_backward_f32(q, k, v, dout, scale=sc)
    assert np.all(dk == 0)
    assert np.abs(dv - np.broadcast_to(dout.sum(axis=2, keepdims=True) / S, v.shape)).max() < 1e-6
    dp = np.einsum("bhld,bhsd->bhls", dout, v)
    ds = (dp - dp.mean(axis=-1, keepdims=True)) / S
    assert np.abs(dq - sc * np.einsum("bhls,bhsd->bhld", ds, k)).max() < 1e-6


def test_invariants():
    """Softmax ignores a shift common to a row's scores, i.e. adding one vector to every key: the columns of dk sum to
    zero over the keys.  And grouped heads equal repeated K/V with the gradients summed over the group."""
    B, Hq, Hkv, L, S, D = 2, 6, 2, 7, 9, 5
    q, k, v, dout = inputs(5, B, Hq, Hkv, L, S, D)
    dq, dk, dv = oracle.sdpa_backward_f32(q, k, v, dout, causal=True)
    assert np.abs(dk.sum(axis=2)).max() < 1e-5
    G = Hq // Hkv
    rq, rk, rv = oracle.sdpa_backward_f32(q, np.repeat(k, G, axis=1), np.repeat(v, G, axis=1), dout, causal=True)
    assert np.abs(rq - dq).max() < 1e-6
    assert np.abs(rk.reshape(B, Hkv, G, S, D).sum(axis=2) - dk).max() < 1e-5
    assert np.abs(rv.reshape(B, Hkv, G, S, D).sum(axis=2) - dv).max() < 1e-5
    # the result does not depend on the thread count
    one = oracle.sdpa_backward_f32(q, k, v, dout, causal=True, nthreads=1)
    assert all(np.array_equal(a, b) for a, b in zip(one, (dq, dk, dv)))


def test_empty_shapes():
    q, k, v, dout = inputs(6, 1, 2, 2, 3, 0, 4)
    dq, dk, dv = oracle.sdpa_backward_f32(q, k, v, dout)
    assert np.all(dq == 0) and dk.size == 0 and dv.size == 0
