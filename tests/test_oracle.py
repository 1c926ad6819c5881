"""Pins the CPU oracle (oracle/sdpa_oracle.c) before anything is checked against it.

Sources of truth, in order: the reference's own known answers (reference test/test_function.cpp:393-419), fixtures
written from the compiled reference (tests/golden/make_fixtures.py), the compiled reference itself when
oracle/_ref is present, the fp64 closed form softmax(QK^T*s + M)V, and invariants that a wrong index, sign or
transposition would break.
"""
import numpy as np
import pytest

from conftest import golden_names, load_golden


def closed_form_f64(q, k, v, causal=False, scale=None, mask=None):
    q, k, v = [np.asarray(t, np.float64) for t in (q, k, v)]
    B, Hq, L, D = q.shape
    Hkv, S = k.shape[1], k.shape[2]
    G = Hq // Hkv
    k = np.repeat(k, G, axis=1)
    v = np.repeat(v, G, axis=1)
    s = np.einsum("bhld,bhsd->bhls", q, k) * (1.0 / np.sqrt(D) if scale is None else scale)
    if causal:
        i, j = np.arange(L)[:, None], np.arange(S)[None, :]
        s = np.where(j <= i, s, -np.inf)
    if mask is not None:
        if mask.dtype == np.uint8 or mask.dtype == np.bool_:
            s = np.where(mask.astype(bool), s, -np.inf)
        else:
            s = s + mask.astype(np.float64)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(axis=-1, keepdims=True)
    return np.einsum("bhls,bhsd->bhld", p, v)


# ---- the reference's own known answers --------------------------------------------------------------------------

REF_PLAIN = [0.9331, 0.6129, 0.9380, 0.6349, 0.4899, 0.7828, 0.4897, 0.7833, 0.6609, 0.6070, 0.6617, 0.5993, 0.2079,
             0.5711, 0.2054, 0.5670]
REF_CAUSAL = [0.9904, 0.8726, 0.9380, 0.6349, 0.4391, 0.9327, 0.4897, 0.7833, 0.6314, 0.8901, 0.6617, 0.5993, 0.0599,
              0.3249, 0.2055, 0.5670]
REF_BOOLMASK = [0.0000, 0.0000, 0.9904, 0.8726, 0.0000, 0.0000, 0.4391, 0.9327, 0.0000, 0.0000, 0.6314, 0.8901,
                0.0000, 0.0000, 0.0599, 0.3249]


def test_reference_known_answers(oracle_mod):
    """reference test/test_function.cpp:404-418, tolerance of its VectorNear (1e-3, test/test.h:17-30)."""
    g = load_golden("kat_plain")
    q, k, v = g["q"], g["k"], g["v"]
    assert np.abs(oracle_mod.sdpa_f32(q, k, v).ravel() - REF_PLAIN).max() < 1e-3
    assert np.abs(oracle_mod.sdpa_f32(q, k, v, causal=True).ravel() - REF_CAUSAL).max() < 1e-3
    m = np.array([[0, 0], [1, 0]], np.uint8)
    y = oracle_mod.sdpa_f32(q, k, v, mask=m).ravel()
    exp = np.array(REF_BOOLMASK)
    live = exp != 0.0
    assert np.abs(y[live] - exp[live]).max() < 1e-3
    # rows whose keys are all hidden: the reference computes 0 * inf = NaN there (its test cannot see it because
    # fabs(NaN - 0) > eps is false); the restatement reproduces the NaN.
    assert np.isnan(y[~live]).all()


def test_softmax_known_answer(oracle_mod):
    """reference test/test_function.cpp:147-155: softmax({1.1,1.2,1.3,1.6}) through a 1-key-dim attention:
    q = [1], k = the logits as [S,1], v = identity -> output row == softmax."""
    logits = np.array([1.1, 1.2, 1.3, 1.6], np.float32)
    q = np.ones((1, 1, 1, 1), np.float32)
    k = logits.reshape(1, 1, 4, 1)
    q4 = np.zeros((1, 1, 1, 4), np.float32)
    k4 = np.zeros((1, 1, 4, 4), np.float32)
    q4[..., 0] = 1.0
    k4[0, 0, :, 0] = logits
    v = np.eye(4, dtype=np.float32).reshape(1, 1, 4, 4)
    y = oracle_mod.sdpa_f32(q4, k4, v, scale=1.0).ravel()
    assert np.abs(y - [0.2010, 0.2221, 0.2455, 0.3314]).max() < 1e-3
    del q, k


# ---- fixtures written from the compiled reference ----------------------------------------------------------------

@pytest.mark.parametrize("name", golden_names())
def test_golden_bit_exact(oracle_mod, name):
    g = load_golden(name)
    y = oracle_mod.sdpa_f32(g["q"], g["k"], g["v"], causal=g["causal"], scale=g["scale"], mask=g["mask"])
    exp = g["out"]
    assert np.array_equal(np.isnan(y), np.isnan(exp))
    ok = ~np.isnan(exp)
    # same compiler family and libm on both sides: expected identical; 1e-6 is the stated bar
    assert np.abs(y[ok] - exp[ok]).max() <= 1e-6
    assert np.array_equal(y[ok], exp[ok])


@pytest.mark.parametrize("name", ["c1_f32_causal", "gqa_hq8_hkv2", "decode_l1_s64", "nonsquare_l7_s4_causal"])
def test_rows_form_matches_full(oracle_mod, name):
    g = load_golden(name)
    if g["mask"] is not None:
        pytest.skip("row form has no mask")
    B, Hq, L, D = g["q"].shape
    rng = np.random.RandomState(3)
    rows = np.stack([rng.randint(0, B, 40), rng.randint(0, Hq, 40), rng.randint(0, L, 40)], axis=1)
    y = oracle_mod.sdpa_rows_f32(g["q"], g["k"], g["v"], rows, causal=g["causal"], scale=g["scale"])
    assert np.array_equal(y, g["out"][rows[:, 0], rows[:, 1], rows[:, 2]])


# ---- the compiled reference, where present ------------------------------------------------------------------------

def _need_ref(oracle_mod):
    if not oracle_mod.have_ref():
        pytest.skip("oracle/_ref/libtt_ref.so not built (needs the reference tree)")


@pytest.mark.parametrize("shape,causal", [
    ((1, 2, 2, 17, 17, 64), True), ((2, 4, 1, 5, 40, 128), False), ((1, 6, 3, 31, 9, 32), True),
    ((1, 1, 1, 1, 1, 8), True), ((1, 2, 2, 64, 64, 128), False),
])
def test_against_compiled_reference(oracle_mod, shape, causal):
    _need_ref(oracle_mod)
    B, Hq, Hkv, L, S, D = shape
    q = oracle_mod.randn(100 + L, 0, (B, Hq, L, D))
    k = oracle_mod.randn(100 + L, 1, (B, Hkv, S, D))
    v = oracle_mod.randn(100 + L, 2, (B, Hkv, S, D))
    a = oracle_mod.sdpa_f32(q, k, v, causal=causal)
    b = oracle_mod.ref_sdpa_f32(q, k, v, causal=causal)
    assert np.array_equal(a, b)
    if Hq != Hkv:  # both GQA spellings of the reference agree (repeatInterleave vs 5-D broadcast matmul)
        assert np.array_equal(b, oracle_mod.ref_sdpa_f32_gqa5d(q, k, v, causal=causal))


def test_threads_do_not_change_bits(oracle_mod):
    q = oracle_mod.randn(7, 0, (2, 4, 50, 64))
    k = oracle_mod.randn(7, 1, (2, 2, 70, 64))
    v = oracle_mod.randn(7, 2, (2, 2, 70, 64))
    assert np.array_equal(oracle_mod.sdpa_f32(q, k, v, nthreads=1), oracle_mod.sdpa_f32(q, k, v, nthreads=5))


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_rounding_against_reference_casts(oracle_mod, dtype):
    _need_ref(oracle_mod)
    x = np.concatenate(
        [oracle_mod.randn(3, i, (50000,)) * s for i, s in enumerate((1e-8, 1e-6, 1e-4, 1e-2, 1, 100, 7e4, 1e30))] +
        [np.array([np.inf, -np.inf, np.nan, 0, -0.0, 65504, 65519.99, 65520, 65536, 2.0**-24, 2.0**-25,
                   2.0**-25 * 1.0001, 2.0**-14, 1.0 + 2.0**-8, 1.0 + 2.0**-7 + 2.0**-8, 1.0 + 2.0**-11,
                   1.0 + 2.0**-10 + 2.0**-11, 3.3895314e38], np.float32)])
    a, _ = oracle_mod.round_to(x, dtype)
    b = oracle_mod.ref_round_trip(x, dtype)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_rounding_f16_against_numpy(oracle_mod):
    x = np.concatenate([oracle_mod.randn(9, i, (50000,)) * s for i, s in enumerate((1e-7, 1e-5, 1e-3, 1, 300))])
    vals, bits = oracle_mod.round_to(x, "f16")
    exp = x.astype(np.float16)
    assert np.array_equal(bits, exp.view(np.uint16))
    assert np.array_equal(vals, exp.astype(np.float32))
    assert np.array_equal(oracle_mod.bits_to_f32(bits, "f16"), vals)


def test_rounding_bf16_ties_and_roundtrip(oracle_mod):
    # ties to even on the 16th bit: 1 + 2^-8 -> 1 (even), 1 + 2^-7 + 2^-8 -> 1 + 2^-6
    x = np.array([1.0 + 2.0**-8, 1.0 + 2.0**-7 + 2.0**-8, 1.0 + 2.0**-8 + 2.0**-20], np.float32)
    vals, bits = oracle_mod.round_to(x, "bf16")
    assert list(vals) == [1.0, 1.0 + 2.0**-6, 1.0 + 2.0**-7]
    allbits = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    f = oracle_mod.bits_to_f32(allbits, "bf16")
    v2, b2 = oracle_mod.round_to(f, "bf16")
    keep = ~np.isnan(f)
    assert np.array_equal(b2[keep], allbits[keep])  # every bf16 value is a fixed point of the rounding


@pytest.mark.parametrize("mshape", [(1, 7), (7,), (2, 1, 5, 7), (2, 4, 5, 7), (2, 1, 1, 7), (1, 4, 5, 1), (4, 1, 7)])
@pytest.mark.parametrize("kind", ["bool", "float"])
def test_broadcast_masks_against_compiled_reference(oracle_mod, mshape, kind):
    _need_ref(oracle_mod)
    B, Hq, Hkv, L, S, D = 2, 4, 2, 5, 7, 8
    q = oracle_mod.randn(31, 0, (B, Hq, L, D))
    k = oracle_mod.randn(31, 1, (B, Hkv, S, D))
    v = oracle_mod.randn(31, 2, (B, Hkv, S, D))
    if kind == "bool":
        m = (np.random.RandomState(len(mshape)).rand(*mshape) > 0.4).astype(np.uint8)
        m[..., 0] = 1
    else:
        m = oracle_mod.randn(32, 3, mshape)
    assert np.array_equal(oracle_mod.sdpa_f32(q, k, v, mask=m), oracle_mod.ref_sdpa_f32(q, k, v, mask=m))


# ---- mathematics ----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("shape,causal", [((2, 4, 2, 19, 23, 32), False), ((1, 4, 4, 40, 40, 64), True),
                                          ((2, 8, 2, 1, 77, 128), False)])
def test_closed_form_fp64(oracle_mod, shape, causal):
    B, Hq, Hkv, L, S, D = shape
    q = oracle_mod.randn(21, 0, (B, Hq, L, D))
    k = oracle_mod.randn(21, 1, (B, Hkv, S, D))
    v = oracle_mod.randn(21, 2, (B, Hkv, S, D))
    y = oracle_mod.sdpa_f32(q, k, v, causal=causal)
    assert np.abs(y - closed_form_f64(q, k, v, causal=causal)).max() < 2e-5


def test_closed_form_masks(oracle_mod):
    g = load_golden("boolmask_l9_s12")
    assert np.abs(g["out"] - closed_form_f64(g["q"], g["k"], g["v"], mask=g["mask"])).max() < 2e-5
    for name in ("floatmask_l9_s12", "boolmask_keypad_b3_s20", "floatmask_b2_h4_l5_s9", "boolmask_h4_1_s11",
                 "floatmask_row_s10"):
        g = load_golden(name)
        assert np.abs(g["out"] - closed_form_f64(g["q"], g["k"], g["v"], mask=g["mask"])).max() < 2e-5, name


def test_invariants(oracle_mod):
    B, H, L, S, D = 1, 2, 12, 12, 16
    q = oracle_mod.randn(31, 0, (B, H, L, D))
    k = oracle_mod.randn(31, 1, (B, H, S, D))
    v = oracle_mod.randn(31, 2, (B, H, S, D))
    # causal row 0 sees only key 0 -> exactly v[0] (visible in reference test_function.cpp:411)
    y = oracle_mod.sdpa_f32(q, k, v, causal=True)
    assert np.array_equal(y[:, :, 0, :], v[:, :, 0, :])
    # identical keys -> uniform weights -> causal output is the running mean of v
    ku = np.broadcast_to(k[:, :, :1, :], k.shape).copy()
    y = oracle_mod.sdpa_f32(q, ku, v, causal=True)
    run = np.cumsum(v.astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert np.abs(y - run).max() < 1e-5
    # v = identity block -> output rows are the softmax weights: non-negative and summing to 1
    vi = np.zeros((B, H, S, S), np.float32)
    vi[:, :, np.arange(S), np.arange(S)] = 1
    qd = oracle_mod.randn(32, 0, (B, H, L, S))
    kd = oracle_mod.randn(32, 1, (B, H, S, S))
    p = oracle_mod.sdpa_f32(qd, kd, vi)
    assert (p >= 0).all() and np.abs(p.sum(-1) - 1).max() < 1e-6
    # permuting the key/value positions does not change a non-causal result (beyond summation order)
    perm = np.random.RandomState(0).permutation(S)
    y0 = oracle_mod.sdpa_f32(q, k, v)
    y1 = oracle_mod.sdpa_f32(q, k[:, :, perm], v[:, :, perm])
    assert np.abs(y0 - y1).max() < 1e-5
    # transposition catch: swapping the roles of L and S operands must change the answer
    assert np.abs(y0 - oracle_mod.sdpa_f32(k, q, v)).max() > 1e-2


def test_prng_moments_and_numpy_restatement(oracle_mod):
    z = oracle_mod.randn(5, 0, (1 << 20,)).astype(np.float64)
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1) < 5e-3
    assert abs((z**3).mean()) < 2e-2 and abs((z**4).mean() - 3) < 5e-2
    assert abs(np.corrcoef(z[:-1], z[1:])[0, 1]) < 5e-3
    # independent numpy restatement of the counter-based construction
    M = (1 << 64) - 1

    def mix(x):
        x = (x + 0x9E3779B97F4A7C15) & M
        x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & M
        x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & M
        return x ^ (x >> 31)

    seed, stream = 1234, 7
    key = mix(seed ^ mix((stream * 0xD1342543DE82EF95 + 0x632BE59BD9B4E019) & M))
    out = oracle_mod.randn(seed, stream, (16,), mul=0.5)
    for i in range(16):
        a, b = mix((key + 2 * i) & M), mix((key + 2 * i + 1) & M)
        u1 = ((a >> 11) + 1.0) * 2.0**-53
        u2 = (b >> 11) * 2.0**-53
        zz = np.sqrt(-2.0 * np.log(u1)) * np.cos(2 * np.pi * u2)
        assert abs(out[i] - np.float32(0.5 * zz)) <= 1e-6 * max(1.0, abs(zz))
    # a stream is a pure function of (seed, stream, index)
    assert np.array_equal(oracle_mod.randn(9, 1, (1000,))[:100], oracle_mod.randn(9, 1, (100,)))
    assert not np.array_equal(oracle_mod.randn(9, 1, (100,)), oracle_mod.randn(9, 2, (100,)))
